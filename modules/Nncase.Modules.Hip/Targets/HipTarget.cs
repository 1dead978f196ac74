// ITarget of the MI355X execution target (interface: src/Nncase.Core/ITarget.cs:26-106).
// With PTQ on, the quantised sub-graphs the importers and the quantiser leave behind (Dequantize -> operator ->
// Quantize, for convolutions, matrix products, residual adds, activations, pooling, concatenation and resizing)
// become hip operators, and connected regions of them are outlined into functions of module kind "hip";
// everything else stays in the stackvm module.
using System;
using System.Collections.Generic;
using System.CommandLine;
using System.CommandLine.Invocation;
using System.Threading.Tasks;
using Microsoft.Extensions.Configuration;
using Nncase.CodeGen;
using Nncase.CodeGen.Hip;
using Nncase.CodeGen.StackVM;
using Nncase.IR;
using Nncase.Passes;
using Nncase.Passes.Rules.Hip;
using Nncase.Quantization;
using Nncase.Runtime.Hip;

namespace Nncase.Targets;

public sealed class HipTarget : ITarget
{
    public string Kind => HipRTModule.Kind;

    public (Command Command, Func<InvocationContext, Command, ITargetCompileOptions> Parser) RegisterCommandAndParser() =>
        (new Command(Kind), (_, _) => DefaultTargetCompileOptions.Instance);

    public void ParseTargetDependentOptions(IConfigurationSection configure)
    {
    }

    public void RegisterTargetInDependentPass(IPassManager passManager, CompileOptions options)
    {
    }

    public void RegisterTargetDependentPass(IPassManager passManager, CompileOptions options)
    {
    }

    public Task<Dictionary<ENode, List<Tuple<List<DataType>, List<List<QuantParam>>, float>>>> BindQuantMethodCosine(ICalibrationDatasetProvider calibrationDataset, List<ENode> rangeOfs, List<ENode> childrenOfRangeOfs, QuantizeOptions quantizeOptions) =>
        Task.FromResult(new Dictionary<ENode, List<Tuple<List<DataType>, List<List<QuantParam>>, float>>>());

    public Task AdaRoundWeights(ICalibrationDatasetProvider calibrationDataset, List<ENode> rangeOfs, List<ENode> childrenOfRangeOfs, QuantizeOptions quantizeOptions) =>
        Task.CompletedTask;

    public void RegisterQuantizePass(IPassManager passManager, CompileOptions options)
    {
    }

    // Runs on the graph the quantiser has already rewritten into Quantize / Dequantize pairs, so the rules see
    // concrete QuantParam constants (a QLinearConv import has them from the start, Onnx/QLinearConv.cs:61-75).
    public void RegisterTargetDependentAfterQuantPass(IPassManager passManager, CompileOptions options)
    {
        if (options.QuantizeOptions.ModelQuantMode != ModelQuantMode.UsePTQ)
        {
            return;
        }

        passManager.AddWithName<DataflowPass>("lowering_hip").Configure(p =>
        {
            p.Add<LowerConv2DToHip>();
            p.Add<LowerMatMulToHip>();
            p.Add<LowerAddToHip>();
            p.Add<LowerReduceMeanToHip>();
            p.Add<LowerReduceWindow2DToHip>();
            p.Add<LowerActivationToHip>();
            p.Add<LowerConcatToHip>();
            p.Add<LowerResizeToHip>();
        });

        // operators that only make sense next to a hip operator: they look at their neighbours, so they run once
        // the sandwiches are gone (and the sandwich rules need the Dequantize calls these would consume)
        passManager.AddWithName<DataflowPass>("lowering_hip_boundary").Configure(p =>
        {
            p.Add<LowerByteConcatToHip>();
            p.Add<LowerResizeToHip>();
            p.Add<LowerReshapeToHip>();
            p.Add<LowerDequantizeToHip>();
            p.Add<LowerQuantizeToHip>();
        });
        passManager.AddWithName<OutlineHipFunctionsPass>("outline_hip");
    }

    public void RegisterTargetDependentBeforeCodeGen(IPassManager passManager, CompileOptions options)
    {
    }

    public IModuleBuilder CreateModuleBuilder(string moduleKind, CompileOptions options) => moduleKind switch
    {
        HipRTModule.Kind => new HipModuleBuilder(),
        Callable.StackVMModuleKind => new StackVMModuleBuilder(),
        _ => throw new NotSupportedException($"{moduleKind} module is not supported."),
    };
}
