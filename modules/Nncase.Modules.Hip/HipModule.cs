// The "hip" target plugin: registers the target and the evaluators of its operators.
// Discovered as an IPlugin (src/Nncase.Core/Hosting/IPlugin.cs:15) by the plugin loader
// (src/Nncase.Compiler/Hosting/PluginLoader.cs:67-98); the K210 module registers itself the same way as an
// application part (modules/Nncase.Modules.K210/K210Module.cs:14-23).
using DryIoc;
using Nncase.Evaluator.Hip;
using Nncase.Hosting;
using Nncase.Targets;

namespace Nncase;

public sealed class HipModule : IPlugin
{
    public void ConfigureServices(IRegistrator registrator)
    {
        registrator.Register<ITarget, HipTarget>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQConv2DEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQMatMulEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQuantizeEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipDequantizeEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQAddEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQGlobalAvgPoolEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQLutEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQConcatEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipResizeNearestEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipQMaxPoolEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipReshapeEvaluator>(reuse: Reuse.Singleton);
        registrator.RegisterManyInterface<HipStoreEvaluator>(reuse: Reuse.Singleton);
    }
}
