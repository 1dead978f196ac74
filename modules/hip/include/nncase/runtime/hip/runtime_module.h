/* Public declarations of the "hip" runtime module for the nncase runtime: the module kind the
 * interpreter resolves (runtime_module::create, src/Native/src/runtime/runtime_loader.cpp:117-128) and
 * the factory the activator returns.  The implementation forwards to the C ABI of libnncase_hip.so
 * (include/nncase_hip.h); it holds no kernels of its own.
 *
 * This file is added to the nncase tree as modules/hip/include/nncase/runtime/hip/runtime_module.h,
 * beside modules/vulkan/include/nncase/runtime/vulkan/runtime_module.h. */
#pragma once
#include <nncase/compiler_defs.h>
#include <nncase/runtime/runtime_module.h>

#define NNCASE_MODULES_HIP_API __attribute__((visibility("default")))

BEGIN_NS_NNCASE_RT_MODULE(hip)

NNCASE_INLINE_VAR constexpr module_kind_t hip_module_kind = to_module_kind("hip");
NNCASE_INLINE_VAR constexpr uint32_t hip_module_version = 1;

/* Section names of a hip module: one operator-record text per function, constants in .rdata
 * (the names every module shares, src/Nncase.CodeGen/CodeGen/SectionManager.cs:24-29). */
NNCASE_INLINE_VAR constexpr char HIP_TEXT_SECTION_NAME[] = ".text";
NNCASE_INLINE_VAR constexpr char HIP_RDATA_SECTION_NAME[] = ".rdata";

NNCASE_MODULES_HIP_API result<std::unique_ptr<runtime_module>> create_hip_runtime_module();

END_NS_NNCASE_RT_MODULE
