// The "hip" target plugin: registers the target and the evaluators of its two operators.
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
    }
}
