// Code generator of the hip module: one operator-record text per function in .text, constants in .rdata.
// The classes follow the split every module builder has (src/Nncase.CodeGen/CodeGen/ModuleBuilder.cs:14-35,
// FunctionBuilder.cs:14-47, LinkableModule.cs:14-50; the K210 and StackVM modules provide the same five).
//
// Function text ("HIPF", version 1), little-endian, all records fixed-size; the runtime reads it with
// nncase_hip_kmodel_load_function:
//   header  32 B : char magic[4]="HIPF"; u32 version, n_tensors, n_ops, input_tensor, output_tensor,
//                  n_outputs (0 = 1; outputs are consecutive tensors), reserved
//   tensor  32 B : u32 typecode, rank (= 4), dims[4] as N, H, W, C; i32 zero_point; f32 scale
//   op     144 B : u32 opcode, n_inputs; i32 inputs[8] (tensor indices, -1 = unused); i32 output; u32 reserved;
//                  u64 rdata0, rdata1 (byte offsets into .rdata, all ones = none); i32 p[16]; f32 f[4]
// Opcodes: 0 quantize, 1 dequantize, 2 conv2d, 3 add, 4 global_avgpool, 5 lut, 6 concat, 7 resize_nearest,
// 8 maxpool, 9 pad_channels, 10 reshape (the output tensor is the input's buffer under other extents).  conv2d: rdata0 = weights (OIHW u8), rdata1 = bias (int32 per output channel);
// p = {out_channels, in_channels / groups, kernel_h, kernel_w, groups, stride_h, stride_w, dilation_h,
// dilation_w, pad_h_before, pad_h_after, pad_w_before, pad_w_after, weights zero point};
// f = {clamp_min, clamp_max, weights scale}.  A matmul is a 1x1 conv2d over [M, 1, 1, K].
using System;
using System.Collections.Generic;
using System.IO;
using System.Linq;
using System.Text;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.Runtime.Hip;

namespace Nncase.CodeGen.Hip;

public sealed class HipModuleBuilder : ModuleBuilder
{
    public override string ModuleKind => HipRTModule.Kind;

    protected override FunctionBuilder CreateFunctionBuilder(uint id) => new HipFunctionBuilder(id, SectionManager);

    protected override ILinkableModule CreateLinkableModule(IReadOnlyList<ILinkableFunction> linkableFunctions) =>
        new HipLinkableModule(linkableFunctions, SectionManager);
}

internal enum HipOpcode : uint
{
    Quantize = 0,
    Dequantize = 1,
    Conv2D = 2,
    Add = 3,
    GlobalAvgPool = 4,
    Lut = 5,
    Concat = 6,
    ResizeNearest = 7,
    MaxPool = 8,
    PadChannels = 9,
    Reshape = 10,
}

internal sealed class HipFunctionBuilder : FunctionBuilder
{
    public const uint TextVersion = 1;
    public const int HeaderBytes = 32;
    public const int TensorBytes = 32;
    public const int OpBytes = 144;
    public const int RdataAlignment = 64;
    private const ulong NoRdata = ulong.MaxValue;

    private readonly List<TensorRecord> _tensors = new();
    private readonly List<OpRecord> _ops = new();
    private uint _output;

    public HipFunctionBuilder(uint id, SectionManager sectionManager)
        : base(id, sectionManager)
    {
    }

    protected override void Compile(BaseFunction callable)
    {
        var fusion = (Fusion)callable;
        if (fusion.Parameters.Length != 1)
        {
            throw new NotSupportedException("a hip function takes one activation");
        }

        var values = new Dictionary<Expr, uint>(ReferenceEqualityComparer.Instance)
        {
            [fusion.Parameters[0]] = AddTensor((TensorType)fusion.Parameters[0].CheckedType!, default),
        };
        _output = Emit(fusion.Body, values);
    }

    protected override void WriteText()
    {
        var w = TextWriter;
        w.Write(Encoding.ASCII.GetBytes("HIPF"));
        w.Write(TextVersion);
        w.Write((uint)_tensors.Count);
        w.Write((uint)_ops.Count);
        w.Write(0u); // input tensor
        w.Write(_output);
        w.Write(0u); // one output
        w.Write(0u);
        foreach (var t in _tensors)
        {
            w.Write(t.TypeCode);
            w.Write(4u);
            foreach (var d in t.Nhwc)
            {
                w.Write((uint)d);
            }

            w.Write(t.QuantParam.ZeroPoint);
            w.Write(t.QuantParam.Scale);
        }

        foreach (var o in _ops)
        {
            w.Write((uint)o.Opcode);
            w.Write((uint)o.Inputs.Length);
            for (int i = 0; i < 8; i++)
            {
                w.Write(i < o.Inputs.Length ? (int)o.Inputs[i] : -1);
            }

            w.Write((int)o.Output);
            w.Write(0u);
            w.Write(o.Rdata0);
            w.Write(o.Rdata1);
            for (int i = 0; i < 16; i++)
            {
                w.Write(i < o.P.Length ? o.P[i] : 0);
            }

            for (int i = 0; i < 4; i++)
            {
                w.Write(i < o.F.Length ? o.F[i] : 0f);
            }
        }
    }

    protected override ILinkableFunction CreateLinkableFunction(uint id, BaseFunction callable, IReadOnlyList<FunctionRef> functionRefs, Stream text) =>
        new HipLinkableFunction(id, callable, functionRefs, text);

    private static uint TypeCode(DataType type) =>
        type == DataTypes.UInt8 ? 0x06u : type == DataTypes.Float32 ? 0x0Bu
        : throw new NotSupportedException($"hip tensors are u8 or f32, not {type}");

    // IR tensors are NCHW (rank 4) or [rows, columns] (rank 2): recorded channels-last
    private uint AddTensor(TensorType type, QuantParam qp)
    {
        var d = type.Shape.ToValueArray();
        int[] nhwc = d.Length switch
        {
            4 => new[] { d[0], d[2], d[3], d[1] },
            2 => new[] { d[0], 1, 1, d[1] },
            _ => throw new NotSupportedException($"hip tensors have rank 2 or 4, not {d.Length}"),
        };
        _tensors.Add(new TensorRecord(TypeCode(type.DType), nhwc, qp.Scale == 0f ? new QuantParam(0, 1f) : qp));
        return (uint)(_tensors.Count - 1);
    }

    private ulong AddConstant(ReadOnlySpan<byte> bytes)
    {
        var writer = SectionManager.GetWriter(WellknownSectionNames.Rdata);
        writer.AlignPosition(RdataAlignment);
        ulong offset = (ulong)writer.Position();
        writer.Write(bytes);
        return offset;
    }

    private uint Emit(Expr expr, Dictionary<Expr, uint> values)
    {
        if (values.TryGetValue(expr, out var known))
        {
            return known;
        }

        if (expr is not Call call)
        {
            throw new NotSupportedException($"unexpected {expr.GetType().Name} in a hip function");
        }

        uint input = Emit(call.Arguments[0], values);
        uint output;
        switch (call.Target)
        {
            case HipQConv2D conv:
                {
                    var weights = ((TensorConst)call.Arguments[1]).Value;
                    var bias = ((TensorConst)call.Arguments[2]).Value;
                    _tensors[(int)input] = _tensors[(int)input] with { QuantParam = conv.InputQuantParam };
                    output = AddTensor((TensorType)call.CheckedType!, conv.OutputQuantParam);
                    var ws = weights.Dimensions;
                    _ops.Add(new OpRecord(
                        HipOpcode.Conv2D,
                        new[] { input },
                        output,
                        AddConstant(weights.BytesBuffer),
                        AddConstant(bias.BytesBuffer),
                        new[]
                        {
                            ws[0], ws[1], ws[2], ws[3], conv.Groups, conv.Strides[0], conv.Strides[1], conv.Dilations[0], conv.Dilations[1],
                            conv.Paddings[0], conv.Paddings[1], conv.Paddings[2], conv.Paddings[3], conv.WeightsQuantParam.ZeroPoint,
                        },
                        new[] { conv.FusedClamp.Min, conv.FusedClamp.Max, conv.WeightsQuantParam.Scale }));
                    break;
                }

            case HipQMatMul matmul:
                {
                    // B[K, N] row-major -> 1x1 convolution weights [N, K, 1, 1]
                    var rhs = ((TensorConst)call.Arguments[1]).Value.ToArray<byte>();
                    var dims = ((TensorConst)call.Arguments[1]).Value.Dimensions;
                    int k = dims[0], n = dims[1];
                    var oihw = new byte[rhs.Length];
                    for (int row = 0; row < k; row++)
                    {
                        for (int col = 0; col < n; col++)
                        {
                            oihw[(col * k) + row] = rhs[(row * n) + col];
                        }
                    }

                    _tensors[(int)input] = _tensors[(int)input] with { QuantParam = matmul.LhsQuantParam };
                    output = AddTensor((TensorType)call.CheckedType!, matmul.OutputQuantParam);
                    _ops.Add(new OpRecord(
                        HipOpcode.Conv2D,
                        new[] { input },
                        output,
                        AddConstant(oihw),
                        NoRdata,
                        new[] { n, k, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, matmul.RhsQuantParam.ZeroPoint },
                        new[] { float.NegativeInfinity, float.PositiveInfinity, matmul.RhsQuantParam.Scale }));
                    break;
                }

            default:
                throw new NotSupportedException($"{call.Target.GetType().Name} is not a hip operator");
        }

        values.Add(expr, output);
        return output;
    }

    private sealed record TensorRecord(uint TypeCode, int[] Nhwc, QuantParam QuantParam);

    private sealed record OpRecord(HipOpcode Opcode, uint[] Inputs, uint Output, ulong Rdata0, ulong Rdata1, int[] P, float[] F);
}

internal sealed class HipLinkableFunction : ILinkableFunction
{
    public HipLinkableFunction(uint id, BaseFunction sourceFunction, IEnumerable<FunctionRef> functionRefs, Stream text)
    {
        Id = id;
        SourceFunction = sourceFunction;
        FunctionRefs = functionRefs;
        Text = text;
    }

    public uint Id { get; }

    public BaseFunction SourceFunction { get; }

    public IEnumerable<FunctionRef> FunctionRefs { get; }

    public Stream Text { get; }

    public IReadOnlyList<ILinkedSection> Sections => Array.Empty<ILinkedSection>();
}

internal sealed class HipLinkableModule : LinkableModule
{
    public HipLinkableModule(IReadOnlyList<ILinkableFunction> functions, SectionManager sectionManager)
        : base(functions, sectionManager)
    {
    }

    protected override ILinkedModule CreateLinkedModule(IReadOnlyList<LinkedFunction> linkedFunctions, Stream text) =>
        new HipLinkedModule(linkedFunctions, text, SectionManager.GetContent(WellknownSectionNames.Rdata));
}

internal sealed class HipLinkedModule : ILinkedModule
{
    public HipLinkedModule(IReadOnlyList<LinkedFunction> functions, Stream text, Stream? rdata)
    {
        Functions = functions;
        Sections = new[]
        {
            new LinkedSection(text, WellknownSectionNames.Text, 0, 8, (ulong)text.Length),
            new LinkedSection(rdata, WellknownSectionNames.Rdata, 0, 8, (ulong)(rdata?.Length ?? 0)),
        };
    }

    public string ModuleKind => HipRTModule.Kind;

    public uint Version => HipRTModule.Version;

    public IReadOnlyList<ILinkedFunction> Functions { get; }

    public IReadOnlyList<ILinkedSection> Sections { get; }
}
