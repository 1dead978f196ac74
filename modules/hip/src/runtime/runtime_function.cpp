/* One function of a hip module.
 *
 * initialize_core takes the function's slice of the module's .text section -- function_header::entrypoint
 * and text_size, exactly as the stackvm function does (src/Native/src/runtime/stackvm/runtime_function.cpp:31-36)
 * -- and hands it, with the module's .rdata, to nncase_hip_kmodel_load_function: the library uploads and
 * pre-packs the constants, allocates one device buffer per tensor, records the operator list and captures
 * it as a HIP graph.
 *
 * invoke_core is what EXTCALL reaches (src/Native/src/runtime/stackvm/ops/control.cpp:25-75).  The
 * compiler emits hip functions as prim functions: the caller allocates the outputs and passes them
 * behind the inputs (control.cpp:49-68), so parameters = [input, output 0, output 1, ...]; a plain function
 * (one parameter) returns its single result instead.  Host tensors
 * are copied in and out around the replay; a caller that keeps activations on the device passes
 * device-backed buffers instead and the copies become device-to-device. */
#include "runtime_function.h"
#include <nncase/runtime/error.h>
#include <nncase/runtime/host_buffer.h>
#include <nncase/runtime/runtime_tensor.h>
#include <nncase/runtime/util.h>

using namespace nncase;
using namespace nncase::runtime;
using namespace nncase::runtime::hip;

namespace {
size_t typecode_bytes(int32_t dtype) noexcept {
    switch (dtype) {
    case NNCASE_HIP_DT_I8:
    case NNCASE_HIP_DT_U8:
        return 1;
    case NNCASE_HIP_DT_I16:
    case NNCASE_HIP_DT_F16:
        return 2;
    case NNCASE_HIP_DT_I32:
    case NNCASE_HIP_DT_F32:
        return 4;
    default:
        return 0;
    }
}
} // namespace

hip_runtime_function::~hip_runtime_function() {
    if (kmodel_)
        (void)nncase_hip_kmodel_destroy(kmodel_); // drains the stream, then frees buffers, constants and the graph
}

hip_runtime_module &hip_runtime_function::module() const noexcept {
    return static_cast<hip_runtime_module &>(runtime_function::module());
}

result<hip_runtime_function::device_tensor> hip_runtime_function::describe(int32_t which) noexcept {
    device_tensor t;
    int32_t dtype = 0, dims[4] = {0, 0, 0, 0};
    hip_try(nncase_hip_kmodel_tensor(kmodel_, which, &t.ptr, &dtype, dims));
    t.bytes = typecode_bytes(dtype) * (size_t)dims[0] * (size_t)dims[1] * (size_t)dims[2] * (size_t)dims[3];
    CHECK_WITH_ERR(t.ptr && t.bytes, nncase_errc::datatype_mismatch);
    return ok(t);
}

result<void> hip_runtime_function::initialize_core(runtime_function_init_context &context) noexcept {
    auto &mod = module();
    const auto &header = context.header();
    CHECK_WITH_ERR(header.entrypoint <= mod.text().size() && header.text_size <= mod.text().size() - header.entrypoint,
                   std::errc::result_out_of_range);
    auto text = mod.text().subspan(header.entrypoint, header.text_size);
    hip_try(nncase_hip_kmodel_load_function(mod.ctx(), text.data(), text.size(), mod.rdata().data(), mod.rdata().size(),
                                            &kmodel_));
    hip_try(nncase_hip_kmodel_function(kmodel_, &function_));
    try_set(input_, describe(NNCASE_HIP_KMODEL_INPUT));
    // a prim function's parameters are its input and then the outputs the caller allocates; a plain function
    // takes the input only and returns its one result
    prim_ = header.parameters > 1;
    const uint32_t n_outputs = prim_ ? header.parameters - 1 : 1;
    for (uint32_t k = 0; k < n_outputs; k++) {
        try_var(out, describe(NNCASE_HIP_KMODEL_OUTPUT - (int32_t)k));
        outputs_.push_back(out);
    }
    hip_try(nncase_hip_function_capture(function_)); // every later invoke is one hipGraphLaunch
    return ok();
}

result<value_t> hip_runtime_function::invoke_core(gsl::span<value_t> parameters, value_t return_value) noexcept {
    CHECK_WITH_ERR(parameters.size() == (prim_ ? outputs_.size() + 1 : 1), std::errc::invalid_argument);
    auto *ctx = module().ctx();

    try_var(in_tensor, parameters[0].as<tensor>());
    try_var(in_span, get_input_span(in_tensor)); // util.h:195-199: host bytes, mapped for reading
    CHECK_WITH_ERR(in_span.size_bytes() == input_.bytes, nncase_errc::shape_mismatch);
    hip_try(nncase_hip_memcpy_h2d(ctx, input_.ptr, in_span.data(), input_.bytes));

    hip_try(nncase_hip_function_invoke(function_));

    auto download = [&](tensor dst, const device_tensor &src) -> result<void> {
        try_var(out_span, get_output_span(dst)); // util.h:178-183: host bytes, mapped for writing
        CHECK_WITH_ERR(out_span.size_bytes() == src.bytes, nncase_errc::shape_mismatch);
        hip_try(nncase_hip_memcpy_d2h(ctx, out_span.data(), src.ptr, src.bytes)); // blocks until the stream has drained
        return ok();
    };
    if (prim_) {
        for (size_t k = 0; k < outputs_.size(); k++) {
            try_var(out_tensor, parameters[k + 1].as<tensor>());
            try_(download(out_tensor, outputs_[k]));
        }
        // the caller pushes the tensors it allocated (control.cpp:63-68) and ignores the returned value
        return ok(parameters[1]);
    }
    tensor out;
    if (!return_value.empty()) {
        try_set(out, return_value.as<tensor>());
    } else { // allocate the declared return type, as EXTCALL does for prim outputs (control.cpp:52-60)
        try_var(ttype, return_type().as<tensor_type>());
        CHECK_WITH_ERR(ttype->shape().is_fixed(), std::errc::invalid_argument);
        dims_t dims;
        for (auto &d : ttype->shape())
            dims.push_back(d.fixed_value());
        try_set(out, runtime::detail::create(ttype->dtype(), dims));
    }
    try_(download(out, outputs_[0]));
    return ok(value_t(out));
}
