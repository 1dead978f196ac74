// Evaluators of the two hip operators: Evaluate() runs the operator on the device through the C ABI, so the
// compiler's evaluator, its PTQ calibration and the dumped per-layer results all see the bytes the kmodel
// will produce.  Tensors cross the boundary as the IR holds them (NCHW, OIHW); the library works channels-last,
// so activations are transposed on the device around the call.
using System;
using Nncase.CostModel;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.Runtime.Hip.Interop;

namespace Nncase.Evaluator.Hip;

internal static class HipDevice
{
    [ThreadStatic]
    private static HipContext? _context;

    // the library keeps one context per host thread and takes no locks
    public static HipContext Context => _context ??= new HipContext();

    public static int TypeCode(DataType type) =>
        type == DataTypes.UInt8 ? 0x06 : type == DataTypes.Float32 ? 0x0B
        : throw new NotSupportedException($"hip operators write u8 or f32, not {type}");
}

public sealed class HipQConv2DEvaluator : IEvaluator<HipQConv2D>, ITypeInferencer<HipQConv2D>, ICostEvaluator<HipQConv2D>
{
    public unsafe IValue Visit(IEvaluateContext context, HipQConv2D conv)
    {
        var input = context.GetArgumentValueAsTensor<byte>(conv, HipQConv2D.Input);
        var weights = context.GetArgumentValueAsTensor<byte>(conv, HipQConv2D.Weights);
        var bias = context.GetArgumentValueAsTensor<int>(conv, HipQConv2D.Bias);
        var outType = (TensorType)context.CurrentCall.CheckedType;
        var (n, c, h, w) = (input.Dimensions[0], input.Dimensions[1], input.Dimensions[2], input.Dimensions[3]);
        var outDims = outType.Shape.ToValueArray();
        int outElem = conv.OutputType == DataTypes.UInt8 ? 1 : 4;
        nuint inBytes = (nuint)input.Length;
        nuint outBytes = (nuint)(outDims[0] * outDims[1] * outDims[2] * outDims[3] * outElem);

        var ctx = HipDevice.Context;
        IntPtr ctxHandle = ctx.DangerousGetHandle();
        IntPtr xNchw = ctx.Alloc(inBytes), xNhwc = ctx.Alloc(inBytes), yNhwc = ctx.Alloc(outBytes), yNchw = ctx.Alloc(outBytes);
        IntPtr packed = IntPtr.Zero;
        try
        {
            var desc = new HipConv2DDesc
            {
                InChannels = c,
                OutChannels = weights.Dimensions[0],
                KernelH = weights.Dimensions[2],
                KernelW = weights.Dimensions[3],
                Groups = conv.Groups,
                WQp = new HipQuantParam(conv.WeightsQuantParam),
                ExpectedPixels = (long)outDims[0] * outDims[2] * outDims[3],
            };
            fixed (byte* wp = weights.Buffer.Span)
            fixed (int* bp = bias.Buffer.Span)
            {
                // the library copies and re-lays-out the constants: the pins end with this call
                ctx.Check(NativeMethods.nncase_hip_qconv2d_prepack(ctxHandle, desc, wp, bp, out packed), "nncase_hip_qconv2d_prepack");
            }

            fixed (byte* xp = input.Buffer.Span)
            {
                ctx.Check(NativeMethods.nncase_hip_memcpy_h2d(ctxHandle, xNchw, xp, inBytes), "nncase_hip_memcpy_h2d");
            }

            ctx.Check(NativeMethods.nncase_hip_nchw_to_nhwc(ctxHandle, xNchw, xNhwc, 1, n, c, h, w), "nncase_hip_nchw_to_nhwc");
            var args = new HipConv2DArgs
            {
                Batch = n,
                InH = h,
                InW = w,
                StrideH = conv.Strides[0],
                StrideW = conv.Strides[1],
                DilationH = conv.Dilations[0],
                DilationW = conv.Dilations[1],
                PadHBefore = conv.Paddings[0],
                PadHAfter = conv.Paddings[1],
                PadWBefore = conv.Paddings[2],
                PadWAfter = conv.Paddings[3],
                XQp = new HipQuantParam(conv.InputQuantParam),
                YQp = new HipQuantParam(conv.OutputQuantParam),
                ClampMin = conv.FusedClamp.Min,
                ClampMax = conv.FusedClamp.Max,
                OutDType = HipDevice.TypeCode(conv.OutputType),
                ResidualDev = IntPtr.Zero,
            };
            ctx.Check(NativeMethods.nncase_hip_qconv2d(ctxHandle, xNhwc, packed, yNhwc, args), "nncase_hip_qconv2d");
            ctx.Check(NativeMethods.nncase_hip_nhwc_to_nchw(ctxHandle, yNhwc, yNchw, outElem, outDims[0], outDims[1], outDims[2], outDims[3]), "nncase_hip_nhwc_to_nchw");

            var result = new byte[(int)outBytes];
            fixed (byte* rp = result)
            {
                ctx.Check(NativeMethods.nncase_hip_memcpy_d2h(ctxHandle, rp, yNchw, outBytes), "nncase_hip_memcpy_d2h"); // drains the stream
            }

            return Value.FromTensor(Tensor.FromBytes(conv.OutputType, result, outDims));
        }
        finally
        {
            if (packed != IntPtr.Zero)
            {
                NativeMethods.nncase_hip_weights_destroy(ctxHandle, packed);
            }

            ctx.Free(xNchw);
            ctx.Free(xNhwc);
            ctx.Free(yNhwc);
            ctx.Free(yNchw);
        }
    }

    public IRType Visit(ITypeInferenceContext context, HipQConv2D target)
    {
        var input = context.CheckArgumentType<TensorType>(target, HipQConv2D.Input);
        var weights = context.CheckArgumentType<TensorType>(target, HipQConv2D.Weights);
        var paddings = Tensor.From(new[] { target.Paddings[0], target.Paddings[1], target.Paddings[2], target.Paddings[3] }, new[] { 2, 2 });
        var shape = (TensorType)TypeInference.Conv2DType(input, weights, target.Strides, paddings, target.Dilations, target.Groups);
        return shape with { DType = target.OutputType };
    }

    public Cost Visit(ICostEvaluateContext context, HipQConv2D target)
    {
        var input = context.GetArgumentType<TensorType>(target, HipQConv2D.Input);
        var weights = context.GetArgumentType<TensorType>(target, HipQConv2D.Weights);
        var output = context.GetReturnType<TensorType>();
        var macs = (uint)(weights.Shape[1].FixedValue * weights.Shape[2].FixedValue * weights.Shape[3].FixedValue);
        return new()
        {
            [CostFactorNames.MemoryLoad] = CostUtility.GetMemoryAccess(input) + CostUtility.GetMemoryAccess(weights),
            [CostFactorNames.MemoryStore] = CostUtility.GetMemoryAccess(output),

            // one MFMA instruction retires 16 x 16 x 64 int8 MACs; 1024 of them issue at once on the device
            [CostFactorNames.CPUCycles] = CostUtility.GetCPUCycles(output, macs * 2) / (16 * 16 * 64 * 2 * 1024 / 16),
        };
    }
}

public sealed class HipQMatMulEvaluator : IEvaluator<HipQMatMul>, ITypeInferencer<HipQMatMul>, ICostEvaluator<HipQMatMul>
{
    public unsafe IValue Visit(IEvaluateContext context, HipQMatMul matmul)
    {
        var lhs = context.GetArgumentValueAsTensor<byte>(matmul, HipQMatMul.Lhs);
        var rhs = context.GetArgumentValueAsTensor<byte>(matmul, HipQMatMul.Rhs);
        int k = rhs.Dimensions[0], nCols = rhs.Dimensions[1];
        int m = (int)(lhs.Length / k); // leading dimensions of the left operand are stacked rows
        int outElem = matmul.OutputType == DataTypes.UInt8 ? 1 : 4;
        nuint outBytes = (nuint)((long)m * nCols * outElem);

        var ctx = HipDevice.Context;
        IntPtr ctxHandle = ctx.DangerousGetHandle();
        IntPtr a = ctx.Alloc((nuint)lhs.Length), y = ctx.Alloc(outBytes);
        IntPtr packed = IntPtr.Zero;
        try
        {
            fixed (byte* bp = rhs.Buffer.Span)
            {
                ctx.Check(NativeMethods.nncase_hip_qmatmul_prepack(ctxHandle, bp, k, nCols, new HipQuantParam(matmul.RhsQuantParam), null, m, out packed), "nncase_hip_qmatmul_prepack");
            }

            fixed (byte* ap = lhs.Buffer.Span)
            {
                ctx.Check(NativeMethods.nncase_hip_memcpy_h2d(ctxHandle, a, ap, (nuint)lhs.Length), "nncase_hip_memcpy_h2d");
            }

            var args = new HipMatMulArgs
            {
                M = m,
                AQp = new HipQuantParam(matmul.LhsQuantParam),
                YQp = new HipQuantParam(matmul.OutputQuantParam),
                ClampMin = float.NegativeInfinity,
                ClampMax = float.PositiveInfinity,
                OutDType = HipDevice.TypeCode(matmul.OutputType),
            };
            ctx.Check(NativeMethods.nncase_hip_qmatmul(ctxHandle, a, packed, y, args), "nncase_hip_qmatmul");
            var result = new byte[(int)outBytes];
            fixed (byte* rp = result)
            {
                ctx.Check(NativeMethods.nncase_hip_memcpy_d2h(ctxHandle, rp, y, outBytes), "nncase_hip_memcpy_d2h");
            }

            var outDims = ((TensorType)context.CurrentCall.CheckedType).Shape.ToValueArray();
            return Value.FromTensor(Tensor.FromBytes(matmul.OutputType, result, outDims));
        }
        finally
        {
            if (packed != IntPtr.Zero)
            {
                NativeMethods.nncase_hip_weights_destroy(ctxHandle, packed);
            }

            ctx.Free(a);
            ctx.Free(y);
        }
    }

    public IRType Visit(ITypeInferenceContext context, HipQMatMul target)
    {
        var lhs = context.CheckArgumentType<TensorType>(target, HipQMatMul.Lhs);
        var rhs = context.CheckArgumentType<TensorType>(target, HipQMatMul.Rhs);
        var shape = (TensorType)TypeInference.MatMulType(lhs, rhs);
        return shape with { DType = target.OutputType };
    }

    public Cost Visit(ICostEvaluateContext context, HipQMatMul target)
    {
        var lhs = context.GetArgumentType<TensorType>(target, HipQMatMul.Lhs);
        var rhs = context.GetArgumentType<TensorType>(target, HipQMatMul.Rhs);
        var output = context.GetReturnType<TensorType>();
        return new()
        {
            [CostFactorNames.MemoryLoad] = CostUtility.GetMemoryAccess(lhs) + CostUtility.GetMemoryAccess(rhs),
            [CostFactorNames.MemoryStore] = CostUtility.GetMemoryAccess(output),
            [CostFactorNames.CPUCycles] = CostUtility.GetCPUCycles(output, (uint)rhs.Shape[0].FixedValue * 2) / (16 * 16 * 64 * 2 * 1024 / 16),
        };
    }
}
