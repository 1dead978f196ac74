// Pre-packed constant block shared by the u8/u8 convolution / matmul kernels.
#pragma once

#include "common.hpp"

struct nncase_hip_weights {
    enum Kind { kIgemm = 0, kDepthwise = 1 };
    int kind = kIgemm;
    int in_channels = 0, out_channels = 0, kernel_h = 0, kernel_w = 0, groups = 1;
    int g_ic = 0, g_oc = 0; // channels per group
    int k = 0;              // reduction length per group: kernel_h * kernel_w * g_ic
    int ksteps = 0;         // ceil(k / 64)
    int tiles = 0;          // 16-channel MFMA tiles per channel chunk (T)
    int nchunks = 0;        // channel chunks per group
    int kc_steps = 0;       // k-steps staged in LDS at a time
    int32_t zw = 0;
    float sw = 1.f;
    // igemm: [groups][nchunks][ksteps][tiles] fragments of 1024 bytes (s8, MFMA operand order)
    // depthwise: [kernel_h * kernel_w][channels] int16 (w - zw)
    void *d_packed = nullptr;
    int32_t *d_wsum = nullptr; // igemm: sum_k (w ^ 0x80 as s8) per out channel; depthwise: sum_t (w - zw)
    int32_t *d_bias = nullptr; // [out_channels]
    size_t packed_bytes = 0;
};

namespace nnhip {

// Output forms of the conv / matmul epilogue.
enum OutMode { kOutU8 = 0, kOutI32 = 1, kOutF32 = 2 };

struct Epilogue {
    float mult;   // sx * sw
    float lo, hi; // fused clamp on the fp32 value
    float sy, zy; // output quantisation
    int out_mode;
};

int launch_qconv_igemm(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                       const nncase_hip_conv2d_args_t *a, int out_h, int out_w);
int launch_qconv_depthwise(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                           const nncase_hip_conv2d_args_t *a, int out_h, int out_w);

// Writes the name of the kernel a conv with these weights / arguments launches.
void describe_conv_kernel(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *a, char *buf, size_t cap);
int igemm_load_mode(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c, int out_h, int out_w);
bool depthwise_uses_3x3(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c);

// Bit-exact requantisation of one fp32 value: sat_u8(rne(y / sy + zy)).
// The saturation is applied to the float (its limits are integers, so it
// commutes with round-half-even); the division is IEEE correctly rounded.
__device__ __forceinline__ uint32_t requant_u8(float y, float sy, float zy) {
    float t = y / sy + zy;
    t = __builtin_fminf(__builtin_fmaxf(t, 0.f), 255.f);
    return (uint32_t)(int32_t)__builtin_rintf(t);
}

__device__ __forceinline__ float clamp_ref(float v, float lo, float hi) {
    return __builtin_fmaxf(__builtin_fminf(v, hi), lo);
}

} // namespace nnhip
