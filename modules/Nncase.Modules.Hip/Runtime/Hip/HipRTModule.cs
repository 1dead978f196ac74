// Module kind and version written into the kmodel's module header
// (src/Native/include/nncase/runtime/model.h:57-64); the runtime module checks the version on load.
namespace Nncase.Runtime.Hip;

public static class HipRTModule
{
    public const string Kind = "hip";

    public const uint Version = 1;
}
