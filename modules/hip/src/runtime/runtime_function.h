/* hip_runtime_function: one function of a hip module = one resident operator list of libnncase_hip.so,
 * replayed as a HIP graph. */
#pragma once
#include "runtime_module.h"
#include <nncase/runtime/runtime_function.h>
#include <vector>

BEGIN_NS_NNCASE_RT_MODULE(hip)

class hip_runtime_function final : public runtime_function {
  public:
    using runtime_function::runtime_function;
    ~hip_runtime_function() override;

    hip_runtime_module &module() const noexcept;

  protected:
    result<void> initialize_core(runtime_function_init_context &context) noexcept override;
    result<value_t> invoke_core(gsl::span<value_t> parameters, value_t return_value) noexcept override;

  private:
    struct device_tensor {
        void *ptr = nullptr;
        size_t bytes = 0;
    };
    result<device_tensor> describe(int32_t which) noexcept;

    nncase_hip_kmodel_t *kmodel_ = nullptr; // owns the device buffers, the pre-packed constants and the function
    nncase_hip_function_t *function_ = nullptr;
    bool prim_ = false; // outputs arrive as trailing parameters
    device_tensor input_;
    std::vector<device_tensor> outputs_;
};

END_NS_NNCASE_RT_MODULE
