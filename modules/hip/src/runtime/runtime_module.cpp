/* The "hip" runtime module: what runtime_module::create("hip") returns once the interpreter has
 * dlopen'ed libnncase.simulator.hip.so and called its activator
 * (src/Native/src/runtime/runtime_loader.cpp:72-84,117-128; export names runtime_loader.h:31-32).
 *
 * initialize_before_functions opens the device (no gfx950 device -> load_model fails with the
 * library's -ENODEV) and pins the module's .text and .rdata images; each function then builds itself
 * from its slice of .text (runtime_function.cpp).  After the functions are built the images are
 * dropped: the library has uploaded every constant by then. */
#include "runtime_module.h"
#include "runtime_function.h"
#include <nncase/runtime/error.h>
#include <nncase/runtime/runtime_loader.h>

using namespace nncase;
using namespace nncase::runtime;
using namespace nncase::runtime::hip;

/* Status values of libnncase_hip.so (nncase_hip.h, error block):
 *   [-NNCASE_ERRC_LAST, -1]   an nncase_errc value with the sign flipped (the errno values the library uses are
 *                             all above NNCASE_ERRC_LAST, so the block is unambiguous)
 *   <= -HIP_STATUS_BASE       -(HIP_STATUS_BASE + hipError_t): a failed HIP runtime call, reported as an I/O error
 *   everything else           -errno */
static constexpr int NNCASE_ERRC_LAST = 0x07;
static constexpr int HIP_STATUS_BASE = 0x1000;

std::error_code nncase::runtime::hip::to_error_code(int rc) noexcept {
    if (rc >= -NNCASE_ERRC_LAST)
        return make_error_code(static_cast<nncase_errc>(-rc)); // src/Native/include/nncase/runtime/error.h:21-37
    if (rc <= -HIP_STATUS_BASE)
        return std::make_error_code(std::errc::io_error);
    return std::make_error_code(static_cast<std::errc>(-rc));
}

hip_runtime_module::~hip_runtime_module() {
    functions_clear_before_context(); // functions hold library objects that die with the context
    if (ctx_)
        (void)nncase_hip_ctx_destroy(ctx_);
}

result<void> hip_runtime_module::initialize_before_functions(runtime_module_init_context &context) noexcept {
    CHECK_WITH_ERR(context.header().version == hip_module_version, nncase_errc::invalid_model_version);
    hip_try(nncase_hip_ctx_create(/*device*/ 0, &ctx_));
    try_set(text_, context.get_or_read_section(HIP_TEXT_SECTION_NAME, text_storage_, false));
    auto rdata = context.get_or_read_section(HIP_RDATA_SECTION_NAME, rdata_storage_, false);
    rdata_ = rdata.is_ok() ? std::move(rdata).unwrap() : gsl::span<const gsl::byte>{}; // a module without constants
    return ok();
}

result<void> hip_runtime_module::initialize_after_functions(NNCASE_UNUSED runtime_module_init_context &context) noexcept {
    text_ = {}, rdata_ = {};
    text_storage_ = nullptr, rdata_storage_ = nullptr;
    return ok();
}

result<std::unique_ptr<runtime_function>> hip_runtime_module::create_function() noexcept {
    std::unique_ptr<runtime_function> fn(new (std::nothrow) hip_runtime_function(*this));
    CHECK_WITH_ERR(fn, std::errc::not_enough_memory);
    return ok(std::move(fn));
}

void hip_runtime_module::functions_clear_before_context() noexcept {
    for (auto &f : functions())
        f.reset();
}

result<std::unique_ptr<runtime_module>> nncase::runtime::hip::create_hip_runtime_module() {
    std::unique_ptr<runtime_module> mod(new (std::nothrow) hip_runtime_module());
    CHECK_WITH_ERR(mod, std::errc::not_enough_memory);
    return ok(std::move(mod));
}

extern "C" {
NNCASE_MODULES_HIP_API void RUNTIME_MODULE_ACTIVATOR_NAME(result<std::unique_ptr<runtime_module>> &result) {
    result = create_hip_runtime_module();
}

/* The module registers no CUSCALL handlers: its functions are reached through EXTCALL only. */
NNCASE_MODULES_HIP_API void
RUNTIME_MODULE_COLLECTOR_NAME(result<std::vector<std::pair<std::string, runtime_module::custom_call_type>>> &result) {
    result = ok(std::vector<std::pair<std::string, runtime_module::custom_call_type>>{});
}
}
