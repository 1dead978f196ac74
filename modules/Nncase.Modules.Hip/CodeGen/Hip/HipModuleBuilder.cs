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
// What p, f and the rdata offsets of each opcode hold is the table HipOpLayouts below.  A matmul is a 1x1 conv2d
// over [M, 1, 1, K].  The IR holds activations as NCHW and the kernels run channels-last: the function starts
// with a layout record (NCHW -> NHWC) on its input and ends with one (NHWC -> NCHW) per output, left out where
// the two orders are the same bytes (rank 2, one channel, or a 1 x 1 image).
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
    Layout = 11,
}

/// <summary>Names of the p[] and f[] fields and the number of .rdata offsets of every opcode, in record order.</summary>
internal static class HipOpLayouts
{
    public static readonly IReadOnlyDictionary<HipOpcode, (string[] P, string[] F, int Rdata)> Fields = new Dictionary<HipOpcode, (string[] P, string[] F, int Rdata)>
    {
        [HipOpcode.Quantize] = (new string[0], new string[0], 0),
        [HipOpcode.Dequantize] = (new string[0], new string[0], 0),
        [HipOpcode.Conv2D] = (
            new[] { "out_channels", "group_in_channels", "kernel_h", "kernel_w", "groups", "stride_h", "stride_w", "dilation_h", "dilation_w", "pad_h_before", "pad_h_after", "pad_w_before", "pad_w_after", "weights_zero_point" },
            new[] { "clamp_min", "clamp_max", "weights_scale" },
            2),
        [HipOpcode.Add] = (new string[0], new[] { "clamp_min", "clamp_max" }, 0),
        [HipOpcode.GlobalAvgPool] = (new string[0], new string[0], 0),
        [HipOpcode.Lut] = (new string[0], new string[0], 1),
        [HipOpcode.Concat] = (new string[0], new string[0], 0),
        [HipOpcode.ResizeNearest] = (new[] { "transformation_mode", "nearest_mode" }, new string[0], 0),
        [HipOpcode.MaxPool] = (new[] { "kernel", "stride", "padding" }, new string[0], 0),
        [HipOpcode.PadChannels] = (new string[0], new string[0], 0),
        [HipOpcode.Reshape] = (new string[0], new string[0], 0),
        [HipOpcode.Layout] = (new[] { "to_nchw" }, new string[0], 0),
    };
}

internal sealed class HipFunctionBuilder : FunctionBuilder
{
    public const uint TextVersion = 1;
    public const int HeaderBytes = 32;
    public const int TensorBytes = 32;
    public const int OpBytes = 144;
    public const int RdataAlignment = 64;
    private const ulong NoRdata = ulong.MaxValue;
    private const int HipConcatLimit = 8; // tensor indices in one operator record

    private readonly List<TensorRecord> _tensors = new();
    private readonly List<OpRecord> _ops = new();
    private readonly Dictionary<uint, uint> _layoutTwin = new();
    private uint _output;
    private uint _outputs = 1;

    public HipFunctionBuilder(uint id, SectionManager sectionManager)
        : base(id, sectionManager)
    {
    }

    protected override void Compile(BaseFunction callable)
    {
        // PrimFunction(in, out_0, ...) { HipStore(value_0, out_0); ... } as OutlineHipFunctionsPass builds it
        var function = (TIR.PrimFunction)callable;
        var parameters = function.Parameters.ToArray();
        var stores = function.Body.Fields.ToArray().Select(f => (Call)f).ToArray();
        if (parameters.Length != stores.Length + 1 || stores.Any(c => c.Target is not HipStore))
        {
            throw new NotSupportedException("a hip function takes one activation and stores each of its outputs once");
        }

        var values = new Dictionary<Expr, uint>(ReferenceEqualityComparer.Instance);
        uint input = AddTensor((TensorType)parameters[0].CheckedType!);
        values[parameters[0]] = ChannelsLast(input, toNchw: false);

        var results = new List<uint>();
        foreach (var store in stores)
        {
            uint value = Emit(store.Arguments[0], values);
            uint result = ChannelsLast(value, toNchw: true);
            if (result == input || results.Contains(result))
            {
                throw new NotSupportedException("an output of a hip function is a tensor of its own");
            }

            results.Add(result);
        }

        MoveOutputsLast(results);
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
        w.Write(_outputs == 1 ? 0u : _outputs);
        w.Write(0u);
        foreach (var t in _tensors)
        {
            w.Write(t.TypeCode);
            w.Write(4u);
            foreach (var d in t.Nhwc)
            {
                w.Write((uint)d);
            }

            w.Write(t.QuantParam?.ZeroPoint ?? 0);
            w.Write(t.QuantParam?.Scale ?? 1f);
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
    private uint AddTensor(TensorType type, QuantParam? qp = null)
    {
        var d = type.Shape.ToValueArray();
        int[] nhwc = d.Length switch
        {
            4 => new[] { d[0], d[2], d[3], d[1] },
            2 => new[] { d[0], 1, 1, d[1] },
            _ => throw new NotSupportedException($"hip tensors have rank 2 or 4, not {d.Length}"),
        };
        return AddTensor(TypeCode(type.DType), nhwc, qp);
    }

    private uint AddTensor(uint typeCode, int[] nhwc, QuantParam? qp)
    {
        _tensors.Add(new TensorRecord(typeCode, nhwc, qp));
        return (uint)(_tensors.Count - 1);
    }

    // A tensor's QuantParam is known from the operator that writes it or from the first one that reads it; the
    // two ends of a layout record share it.  Two operators that disagree describe a graph the rules should not
    // have lowered.
    private void SetQuantParam(uint tensor, QuantParam qp)
    {
        var known = _tensors[(int)tensor].QuantParam;
        if (known is QuantParam k && (k.ZeroPoint != qp.ZeroPoint || k.Scale != qp.Scale))
        {
            throw new NotSupportedException($"tensor {tensor} is read as ({qp.ZeroPoint}, {qp.Scale}) but written as ({k.ZeroPoint}, {k.Scale})");
        }

        _tensors[(int)tensor] = _tensors[(int)tensor] with { QuantParam = qp };
        if (_layoutTwin.TryGetValue(tensor, out var twin) && _tensors[(int)twin].QuantParam is null)
        {
            SetQuantParam(twin, qp);
        }
    }

    // the same tensor in the other byte order, through a layout record; the tensor itself where both orders agree
    private uint ChannelsLast(uint tensor, bool toNchw)
    {
        var t = _tensors[(int)tensor];
        if (t.Nhwc[3] == 1 || t.Nhwc[1] * t.Nhwc[2] == 1)
        {
            return tensor;
        }

        uint other = AddTensor(t.TypeCode, t.Nhwc, t.QuantParam);
        _layoutTwin[tensor] = other;
        _layoutTwin[other] = tensor;
        AddOp(HipOpcode.Layout, new[] { tensor }, other, p: new[] { toNchw ? 1 : 0 });
        return other;
    }

    // outputs are the last tensors of the table, in the order of the function's output parameters
    private void MoveOutputsLast(List<uint> results)
    {
        var order = Enumerable.Range(0, _tensors.Count).Select(i => (uint)i).Where(i => !results.Contains(i)).Concat(results).ToArray();
        var renumber = new uint[order.Length];
        for (uint position = 0; position < order.Length; position++)
        {
            renumber[order[position]] = position;
        }

        var tensors = order.Select(i => _tensors[(int)i]).ToArray();
        _tensors.Clear();
        _tensors.AddRange(tensors);
        for (int i = 0; i < _ops.Count; i++)
        {
            _ops[i] = _ops[i] with { Inputs = _ops[i].Inputs.Select(t => renumber[t]).ToArray(), Output = renumber[_ops[i].Output] };
        }

        _output = (uint)(order.Length - results.Count);
        _outputs = (uint)results.Count;
    }

    private void AddOp(HipOpcode opcode, uint[] inputs, uint output, ulong rdata0 = NoRdata, ulong rdata1 = NoRdata, int[]? p = null, float[]? f = null)
    {
        var (pNames, fNames, rdata) = HipOpLayouts.Fields[opcode];
        p ??= Array.Empty<int>();
        f ??= Array.Empty<float>();
        int offsets = (rdata0 != NoRdata ? 1 : 0) + (rdata1 != NoRdata ? 1 : 0);
        if (p.Length != pNames.Length || f.Length != fNames.Length || offsets > rdata || inputs.Length > HipConcatLimit)
        {
            throw new InvalidOperationException($"{opcode} record does not follow its layout");
        }

        _ops.Add(new OpRecord(opcode, inputs, output, rdata0, rdata1, p, f));
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

        if (expr is not Call { Target: IHipOp } call)
        {
            throw new NotSupportedException($"unexpected {expr.GetType().Name} in a hip function");
        }

        var inputs = Passes.OutlineHipFunctionsPass.Activations(call).Select(a => Emit(a, values)).ToArray();
        uint input = inputs[0];
        var type = (TensorType)call.CheckedType!;
        uint output;
        switch (call.Target)
        {
            case HipQConv2D conv:
                output = EmitConv2D(conv, call, input);
                break;

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

                    SetQuantParam(input, matmul.LhsQuantParam);
                    output = AddTensor(type, matmul.OutputQuantParam);
                    AddOp(
                        HipOpcode.Conv2D,
                        new[] { input },
                        output,
                        AddConstant(oihw),
                        NoRdata,
                        new[] { n, k, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, matmul.RhsQuantParam.ZeroPoint },
                        new[] { float.NegativeInfinity, float.PositiveInfinity, matmul.RhsQuantParam.Scale });
                    break;
                }

            case HipQuantize quantize:
                output = AddTensor(type, quantize.QuantParam);
                AddOp(HipOpcode.Quantize, new[] { input }, output);
                break;

            case HipDequantize dequantize:
                SetQuantParam(input, dequantize.QuantParam);
                output = AddTensor(type);
                AddOp(HipOpcode.Dequantize, new[] { input }, output);
                break;

            case HipQAdd add:
                SetQuantParam(inputs[0], add.LhsQuantParam);
                SetQuantParam(inputs[1], add.RhsQuantParam);
                output = AddTensor(type, add.OutputQuantParam);
                AddOp(HipOpcode.Add, inputs, output, f: new[] { add.FusedClamp.Min, add.FusedClamp.Max });
                break;

            case HipQGlobalAvgPool pool:
                SetQuantParam(input, pool.InputQuantParam);
                output = AddTensor(type, pool.OutputQuantParam);
                AddOp(HipOpcode.GlobalAvgPool, new[] { input }, output);
                break;

            case HipQLut lut:
                SetQuantParam(input, lut.InputQuantParam);
                output = AddTensor(type, lut.OutputQuantParam);
                AddOp(HipOpcode.Lut, new[] { input }, output, AddConstant(((TensorConst)call.Arguments[1]).Value.BytesBuffer));
                break;

            case HipQConcat concat:
                {
                    // (0, 1) for every tensor is the byte concatenation of tensors that already share one QuantParam
                    bool bytes = concat.OutputQuantParam.Scale == 1f && concat.OutputQuantParam.ZeroPoint == 0 && concat.InputQuantParams.All(q => q.Scale == 1f && q.ZeroPoint == 0);
                    var shared = _tensors[(int)inputs[0]].QuantParam;
                    for (int i = 0; i < inputs.Length; i++)
                    {
                        if (!bytes)
                        {
                            SetQuantParam(inputs[i], concat.InputQuantParams[i]);
                        }
                        else if (shared is null || !Nullable.Equals(_tensors[(int)inputs[i]].QuantParam, shared))
                        {
                            throw new NotSupportedException("a byte concatenation joins tensors of one QuantParam");
                        }
                    }

                    output = AddTensor(type, bytes ? shared : concat.OutputQuantParam);
                    AddOp(HipOpcode.Concat, inputs, output);
                    break;
                }

            case HipResizeNearest resize:
                output = AddTensor(type, _tensors[(int)input].QuantParam ?? resize.QuantParam);
                AddOp(HipOpcode.ResizeNearest, new[] { input }, output, p: new[] { (int)resize.TransformationMode, (int)resize.NearestMode });
                break;

            case HipQMaxPool pool:
                SetQuantParam(input, pool.InputQuantParam);
                output = AddTensor(type, pool.OutputQuantParam);
                AddOp(HipOpcode.MaxPool, new[] { input }, output, p: new[] { pool.Kernel, pool.Stride, pool.Padding });
                break;

            case HipReshape:
                output = AddTensor(type, _tensors[(int)input].QuantParam);
                AddOp(HipOpcode.Reshape, new[] { input }, output);
                break;

            default:
                throw new NotSupportedException($"{call.Target.GetType().Name} has no record in a hip function");
        }

        values.Add(expr, output);
        return output;
    }

    private uint EmitConv2D(HipQConv2D conv, Call call, uint input)
    {
        var weights = ((TensorConst)call.Arguments[1]).Value;
        var bias = ((TensorConst)call.Arguments[2]).Value;
        var ws = weights.Dimensions.ToArray();
        var bytes = weights.BytesBuffer.ToArray();
        SetQuantParam(input, conv.InputQuantParam);

        // A dense convolution over fewer than four channels (an RGB stem) would gather single bytes: its input is
        // padded to four channels and its weights with their zero point, whose products (w - zero point) vanish
        // whatever the padded bytes are.  (3 x 3 windows of stride 1 are left to the kernel.)
        bool small = conv.Groups == 1 && ws[1] < 4 && !(ws[2] == 3 && ws[3] == 3 && conv.Strides[0] == 1 && conv.Strides[1] == 1);
        if (small)
        {
            var t = _tensors[(int)input];
            uint padded = AddTensor(t.TypeCode, new[] { t.Nhwc[0], t.Nhwc[1], t.Nhwc[2], 4 }, t.QuantParam);
            AddOp(HipOpcode.PadChannels, new[] { input }, padded);
            int taps = ws[2] * ws[3];
            var wide = Enumerable.Repeat((byte)conv.WeightsQuantParam.ZeroPoint, ws[0] * 4 * taps).ToArray();
            for (int o = 0; o < ws[0]; o++)
            {
                Array.Copy(bytes, o * ws[1] * taps, wide, o * 4 * taps, ws[1] * taps);
            }

            (input, bytes, ws[1]) = (padded, wide, 4);
        }

        uint output = AddTensor((TensorType)call.CheckedType!, conv.OutputType == DataTypes.UInt8 ? conv.OutputQuantParam : null);
        AddOp(
            HipOpcode.Conv2D,
            new[] { input },
            output,
            AddConstant(bytes),
            AddConstant(bias.BytesBuffer),
            new[]
            {
                ws[0], ws[1], ws[2], ws[3], conv.Groups, conv.Strides[0], conv.Strides[1], conv.Dilations[0], conv.Dilations[1],
                conv.Paddings[0], conv.Paddings[1], conv.Paddings[2], conv.Paddings[3], conv.WeightsQuantParam.ZeroPoint,
            },
            new[] { conv.FusedClamp.Min, conv.FusedClamp.Max, conv.WeightsQuantParam.Scale });
        return output;
    }

    private sealed record TensorRecord(uint TypeCode, int[] Nhwc, QuantParam? QuantParam);

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
