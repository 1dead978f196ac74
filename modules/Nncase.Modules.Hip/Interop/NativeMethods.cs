// P/Invoke surface of libnncase_hip.so (include/nncase_hip.h), in the style of the simulator's own bindings
// (src/Nncase.Simulator/Runtime/Interop/Native.cs:15-87): sequential PODs with the header's field order and
// types, IntPtr for opaque handles and device pointers, int status codes.
//
// The struct layouts are checked against the header by the kernel library's test suite (it reads the field
// lists below); keep one field per declarator and the header's order.
using System;
using System.Runtime.InteropServices;

namespace Nncase.Runtime.Hip.Interop;

[StructLayout(LayoutKind.Sequential)]
public struct HipQuantParam
{
    public int ZeroPoint;
    public float Scale;

    public HipQuantParam(QuantParam qp)
    {
        ZeroPoint = qp.ZeroPoint;
        Scale = qp.Scale;
    }
}

/// <summary>nncase_hip_conv2d_desc_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipConv2DDesc
{
    public int InChannels;
    public int OutChannels;
    public int KernelH;
    public int KernelW;
    public int Groups;
    public HipQuantParam WQp;
    public long ExpectedPixels;
}

/// <summary>nncase_hip_conv2d_args_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipConv2DArgs
{
    public int Batch;
    public int InH;
    public int InW;
    public int StrideH;
    public int StrideW;
    public int DilationH;
    public int DilationW;
    public int PadHBefore;
    public int PadHAfter;
    public int PadWBefore;
    public int PadWAfter;
    public HipQuantParam XQp;
    public HipQuantParam YQp;
    public float ClampMin;
    public float ClampMax;
    public int OutDType;
    public IntPtr ResidualDev;
    public HipQuantParam ResidualQp;
    public HipQuantParam SumQp;
    public float SumClampMin;
    public float SumClampMax;
    public int OutChannelStride;
    public int OutChannelOffset;
    public int DequantizeOutput;
    public int Reserved;
}

/// <summary>nncase_hip_qblock_desc_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipQBlockDesc
{
    public int InChannels;
    public int MidChannels;
    public int OutChannels;
    public HipQuantParam ExpandWQp;
    public HipQuantParam DwWQp;
    public HipQuantParam ProjectWQp;
}

/// <summary>nncase_hip_qblock_args_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipQBlockArgs
{
    public int Batch;
    public int InH;
    public int InW;
    public int Stride;
    public int PadHBefore;
    public int PadHAfter;
    public int PadWBefore;
    public int PadWAfter;
    public HipQuantParam XQp;
    public HipQuantParam ExpandQp;
    public HipQuantParam DwQp;
    public HipQuantParam YQp;
    public float ExpandClampMin;
    public float ExpandClampMax;
    public float DwClampMin;
    public float DwClampMax;
    public float ClampMin;
    public float ClampMax;
    public int AddInput;
    public HipQuantParam SumQp;
    public float SumClampMin;
    public float SumClampMax;
}

/// <summary>nncase_hip_matmul_args_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipMatMulArgs
{
    public int M;
    public HipQuantParam AQp;
    public HipQuantParam YQp;
    public float ClampMin;
    public float ClampMax;
    public int OutDType;
}

/// <summary>nncase_hip_paged_attn_args_t.</summary>
[StructLayout(LayoutKind.Sequential)]
public struct HipPagedAttnArgs
{
    public int Batch;
    public int NumQHeads;
    public int NumKvHeads;
    public int HeadDim;
    public int BlockSize;
    public int MaxBlocksPerSeq;
    public int NumBlocks;
    public float Scale;
    public int OutDType;
    public int CtxLenOffset;
}

internal static unsafe class NativeMethods
{
    private const string Lib = "nncase_hip";

    [DllImport(Lib)]
    public static extern int nncase_hip_ctx_create(int device, out IntPtr ctx);

    [DllImport(Lib)]
    public static extern int nncase_hip_ctx_destroy(IntPtr ctx);

    [DllImport(Lib)]
    public static extern IntPtr nncase_hip_last_error_string(IntPtr ctx);

    [DllImport(Lib)]
    public static extern int nncase_hip_stream_sync(IntPtr ctx);

    [DllImport(Lib)]
    public static extern int nncase_hip_malloc(IntPtr ctx, nuint bytes, out IntPtr dptr);

    [DllImport(Lib)]
    public static extern int nncase_hip_free(IntPtr ctx, IntPtr dptr);

    [DllImport(Lib)]
    public static extern int nncase_hip_memcpy_h2d(IntPtr ctx, IntPtr dst, void* src, nuint bytes);

    [DllImport(Lib)]
    public static extern int nncase_hip_memcpy_d2h(IntPtr ctx, void* dst, IntPtr src, nuint bytes);

    [DllImport(Lib)]
    public static extern int nncase_hip_nchw_to_nhwc(IntPtr ctx, IntPtr src, IntPtr dst, int elemSize, int n, int c, int h, int w);

    [DllImport(Lib)]
    public static extern int nncase_hip_nhwc_to_nchw(IntPtr ctx, IntPtr src, IntPtr dst, int elemSize, int n, int c, int h, int w);

    [DllImport(Lib)]
    public static extern int nncase_hip_qconv2d_prepack(IntPtr ctx, in HipConv2DDesc desc, byte* weightsOihw, int* bias, out IntPtr weights);

    [DllImport(Lib)]
    public static extern int nncase_hip_weights_destroy(IntPtr ctx, IntPtr weights);

    [DllImport(Lib)]
    public static extern int nncase_hip_qconv2d(IntPtr ctx, IntPtr x, IntPtr weights, IntPtr y, in HipConv2DArgs args);

    [DllImport(Lib)]
    public static extern int nncase_hip_qmatmul_prepack(IntPtr ctx, byte* b, int k, int n, HipQuantParam bQp, int* bias, long expectedRows, out IntPtr weights);

    [DllImport(Lib)]
    public static extern int nncase_hip_qmatmul(IntPtr ctx, IntPtr a, IntPtr weights, IntPtr y, in HipMatMulArgs args);

    [DllImport(Lib)]
    public static extern int nncase_hip_qblock_supported(in HipQBlockDesc desc);

    [DllImport(Lib)]
    public static extern int nncase_hip_qblock_prepack(IntPtr ctx, in HipQBlockDesc desc, byte* wExpand, int* biasExpand, byte* wDw, int* biasDw, byte* wProject, int* biasProject, out IntPtr block);

    [DllImport(Lib)]
    public static extern int nncase_hip_qblock_destroy(IntPtr ctx, IntPtr block);

    [DllImport(Lib)]
    public static extern int nncase_hip_qblock(IntPtr ctx, IntPtr x, IntPtr block, IntPtr y, in HipQBlockArgs args);

    [DllImport(Lib)]
    public static extern int nncase_hip_paged_attention_decode(IntPtr ctx, IntPtr q, IntPtr kCache, IntPtr vCache, IntPtr blockTable, IntPtr ctxLens, IntPtr output, in HipPagedAttnArgs args);
}

/// <summary>
/// One device context per evaluator thread; throws with the library's message on a non-zero status, like
/// src/Nncase.Simulator/Runtime/Interop/ErrorCode.cs:25-31.
/// </summary>
internal sealed class HipContext : SafeHandle
{
    public HipContext(int device = 0)
        : base(IntPtr.Zero, true)
    {
        int rc = NativeMethods.nncase_hip_ctx_create(device, out var ctx);
        if (rc != 0)
        {
            throw new InvalidOperationException($"nncase_hip_ctx_create: status {rc} (is there a gfx950 device and is libnncase_hip.so on the loader path?)");
        }

        SetHandle(ctx);
    }

    public override bool IsInvalid => handle == IntPtr.Zero;

    public void Check(int rc, string what)
    {
        if (rc != 0)
        {
            var message = Marshal.PtrToStringAnsi(NativeMethods.nncase_hip_last_error_string(handle));
            throw new InvalidOperationException($"{what}: status {rc} {message}");
        }
    }

    public IntPtr Alloc(nuint bytes)
    {
        Check(NativeMethods.nncase_hip_malloc(handle, bytes, out var p), "nncase_hip_malloc");
        return p;
    }

    public void Free(IntPtr p) => Check(NativeMethods.nncase_hip_free(handle, p), "nncase_hip_free");

    protected override bool ReleaseHandle() => NativeMethods.nncase_hip_ctx_destroy(handle) == 0;
}
