/* hip_runtime_module: owns the device context of one loaded "hip" module and the two section
 * images its functions are built from. */
#pragma once
#include <nncase/runtime/hip/runtime_module.h>
#include <nncase_hip.h>

BEGIN_NS_NNCASE_RT_MODULE(hip)

/* A status of libnncase_hip.so -> the error_code the runtime reports: [-7, -1] is an nncase_errc value with the
 * sign flipped, -(0x1000 + hipError_t) and below a failed HIP runtime call (std::errc::io_error), anything else
 * a negative errno (nncase_hip.h, error block). */
std::error_code to_error_code(int rc) noexcept;

#define hip_try(x)                                                                                                     \
    do {                                                                                                               \
        int rc_ = (x);                                                                                                 \
        if (rc_ != 0)                                                                                                  \
            return err(::nncase::runtime::hip::to_error_code(rc_));                                                    \
    } while (0)

class hip_runtime_module final : public runtime_module {
  public:
    ~hip_runtime_module() override;

    nncase_hip_ctx_t *ctx() const noexcept { return ctx_; }
    gsl::span<const gsl::byte> text() const noexcept { return text_; }
    gsl::span<const gsl::byte> rdata() const noexcept { return rdata_; }

  protected:
    result<void> initialize_before_functions(runtime_module_init_context &context) noexcept override;
    result<void> initialize_after_functions(runtime_module_init_context &context) noexcept override;
    result<std::unique_ptr<runtime_function>> create_function() noexcept override;

  private:
    void functions_clear_before_context() noexcept;

    nncase_hip_ctx_t *ctx_ = nullptr;
    gsl::span<const gsl::byte> text_, rdata_;
    host_buffer_t text_storage_, rdata_storage_;
};

END_NS_NNCASE_RT_MODULE
