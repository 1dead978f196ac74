/*
 * nncase_hip.h -- C ABI of libnncase_hip.so, the MI355X (gfx950) kernel
 * library behind nncase's `hip` execution target.
 *
 * Conventions, copied from nncase's own pure-C surface
 * (src/Native/include/nncase/api.h:43-110, src/Native/src/api.cpp:25-49):
 *   - every function returns int: 0 on success, a negative value on failure
 *     (-errno for argument / resource errors, -(0x1000 + hipError_t) for HIP
 *     runtime errors, -nncase_errc for datatype/shape mismatches);
 *   - every pointer argument is null-checked (-EINVAL);
 *   - objects handed out are owned by the caller until the matching
 *     *_destroy / *_free call;
 *   - one context per host thread, no internal locking (the reference runtime
 *     is single threaded: src/Native/src/runtime/interpreter.cpp).
 * Kernels are enqueued on the context's HIP stream and the call returns at
 * once; nncase_hip_stream_sync blocks until the stream has drained.
 *
 * Tensors on this boundary are dense, activations are NHWC (channels
 * contiguous) unless a function says otherwise; weights are handed over in
 * nncase's OIHW order on the HOST and re-laid-out once by the *_prepack calls.
 * Data-type arguments use nncase's typecodes
 * (src/Native/include/nncase/runtime/typecodes.def).
 */
#ifndef NNCASE_HIP_H
#define NNCASE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNCASE_HIP_API __attribute__((visibility("default")))

/* nncase typecodes used on this boundary (typecodes.def). */
enum {
    NNCASE_HIP_DT_I8 = 0x02,
    NNCASE_HIP_DT_I16 = 0x03,
    NNCASE_HIP_DT_I32 = 0x04,
    NNCASE_HIP_DT_U8 = 0x06,
    NNCASE_HIP_DT_F16 = 0x0A,
    NNCASE_HIP_DT_F32 = 0x0B
};

/* Error values beyond errno; returned negated.  The first block mirrors
 * nncase_errc (src/Native/include/nncase/runtime/error.h:21-37).  The errno
 * values the library returns are all above it (ENOMEM 12, EFAULT 14, EBUSY 16,
 * ENODEV 19, EINVAL 22, ENOSPC 28, ...): a status in [-7, -1] is always an
 * nncase_errc, so a caller can map every status back without ambiguity. */
enum {
    NNCASE_HIP_ERR_INVALID_MODEL_IDENTIFIER = 0x01,
    NNCASE_HIP_ERR_INVALID_MODEL_VERSION = 0x03,
    NNCASE_HIP_ERR_RUNTIME_NOT_FOUND = 0x04,
    NNCASE_HIP_ERR_DATATYPE_MISMATCH = 0x05,
    NNCASE_HIP_ERR_SHAPE_MISMATCH = 0x06,
    NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION = 0x07,
    NNCASE_HIP_ERR_HIP_BASE = 0x1000 /* -(0x1000 + hipError_t) */
};

/* Mirrors quant_param_t (src/Native/include/nncase/runtime/simple_types.h:157-165). */
typedef struct nncase_hip_quant_param {
    int32_t zero_point;
    float scale;
} nncase_hip_quant_param_t;

typedef struct nncase_hip_ctx nncase_hip_ctx_t;         /* device + stream      */
typedef struct nncase_hip_weights nncase_hip_weights_t; /* pre-packed constants */

/* ---- library / context ------------------------------------------------- */

/* Library version, major << 16 | minor. */
NNCASE_HIP_API int nncase_hip_version(void);

/* Creates a context on HIP device `device` with a stream of its own.  Fails
 * with -ENODEV when the device is not a gfx950 part.  Counterpart of
 * nncase_interp_create (api.h:77). */
NNCASE_HIP_API int nncase_hip_ctx_create(int device, nncase_hip_ctx_t **ctx);
NNCASE_HIP_API int nncase_hip_ctx_destroy(nncase_hip_ctx_t *ctx);
/* For hosts that keep several contexts busy at once (one per request in flight, as one interpreter per request
 * with the reference): HIP multiplexes streams over at most GPU_MAX_HW_QUEUES hardware queues (4 by default) — a new
 * stream opens a new queue until that many exist and joins the least shared one after that — and kernels of
 * streams that share a queue run one after the other.  This call creates that many idle streams on the device, once
 * per process, so that the streams of contexts created AFTER it land on the hardware queues in turn, one each for
 * the first GPU_MAX_HW_QUEUES of them.  Returns the number of hardware queues (> 0) or a negative status.
 * (No counterpart in the reference, whose interpreters are CPU threads.) */
NNCASE_HIP_API int nncase_hip_fill_queue_pool(int device);
/* Destroys the idle streams nncase_hip_fill_queue_pool created on `device` (for a host that unloads the library or
 * is done with overlapping requests); contexts created afterwards share hardware queues as HIP deals them out.
 * Returns the number of streams destroyed (0: the pool was not filled), or a negative status.  No counterpart in
 * the reference (its CPU runtime has no queues). */
NNCASE_HIP_API int nncase_hip_release_queue_pool(int device);

/* The hipStream_t the context enqueues on (so a caller can record events on
 * it), and a way to make the context use a caller-owned stream instead. */
NNCASE_HIP_API int nncase_hip_ctx_get_stream(nncase_hip_ctx_t *ctx, void **hip_stream);
NNCASE_HIP_API int nncase_hip_ctx_set_stream(nncase_hip_ctx_t *ctx, void *hip_stream);

/* Text of the last error recorded on this context ("" when none); the
 * pointer stays valid until the next failing call on the context. */
NNCASE_HIP_API const char *nncase_hip_last_error_string(nncase_hip_ctx_t *ctx);

/* Device properties the benchmark reports: compute units, clock in kHz. */
NNCASE_HIP_API int nncase_hip_device_info(nncase_hip_ctx_t *ctx, int *compute_units,
                                          int *clock_khz, size_t *hbm_bytes);

/* ---- device memory (counterpart of nncase_buffer_allocator_alloc /
 *      nncase_host_buffer_map, api.h:59-67; here the memory is HBM) -------- */
NNCASE_HIP_API int nncase_hip_malloc(nncase_hip_ctx_t *ctx, size_t bytes, void **dptr);
NNCASE_HIP_API int nncase_hip_free(nncase_hip_ctx_t *ctx, void *dptr);
NNCASE_HIP_API int nncase_hip_memcpy_h2d(nncase_hip_ctx_t *ctx, void *dst_dev, const void *src_host, size_t bytes);
NNCASE_HIP_API int nncase_hip_memcpy_d2h(nncase_hip_ctx_t *ctx, void *dst_host, const void *src_dev, size_t bytes);
NNCASE_HIP_API int nncase_hip_memset(nncase_hip_ctx_t *ctx, void *dptr, int byte, size_t bytes);
NNCASE_HIP_API int nncase_hip_stream_sync(nncase_hip_ctx_t *ctx);

/* ---- quantize / dequantize --------------------------------------------- */

/* q = sat_T((int32) rne(x / scale + (float)zero_point)), T in {u8, i8, i16}.
 * Replaces kernels::stackvm::quantize
 * (src/Native/src/kernels/stackvm/tensor_ops.cpp:681-695 ->
 *  reference/quantize.cpp:29-43, optimized/quantize.cpp:58-68).
 * in_dtype is f32 or f16; `count` elements, contiguous. */
NNCASE_HIP_API int nncase_hip_quantize(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                       int out_dtype, size_t count, nncase_hip_quant_param_t qp);

/* y = ((float)q - (float)zero_point) * scale, q in {u8, i8, i16, i32},
 * out_dtype f32 or f16 (f16: the f32 value rounded to nearest even).
 * Replaces kernels::stackvm::dequantize
 * (tensor_ops.cpp:268-283 -> reference/dequantize.cpp:29-39). */
NNCASE_HIP_API int nncase_hip_dequantize(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                         int out_dtype, size_t count, nncase_hip_quant_param_t qp);

/* The same two operators on strided operands, as the reference's kernels take them
 * (in_shape, in_strides, out_strides; reference/quantize.cpp:29-47, dequantize.cpp:29-44,
 * called with the tensors' own strides from tensor_ops.cpp:268-283,681-695): element `index`
 * is read at sum(index[d] * in_strides[d]) and written at sum(index[d] * out_strides[d]),
 * strides in elements, rank 1..6.  Elements the output strides skip are left untouched. */
NNCASE_HIP_API int nncase_hip_quantize_strided(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                               int out_dtype, int32_t rank, const int64_t *shape,
                                               const int64_t *in_strides, const int64_t *out_strides,
                                               nncase_hip_quant_param_t qp);
NNCASE_HIP_API int nncase_hip_dequantize_strided(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                                 int out_dtype, int32_t rank, const int64_t *shape,
                                                 const int64_t *in_strides, const int64_t *out_strides,
                                                 nncase_hip_quant_param_t qp);

/* ---- u8/u8 convolution and matmul --------------------------------------
 *
 * acc[p, oc] = bias[oc] + sum_{ky,kx,ic} (x - zx) * (w - zw)          (int32)
 * out_dtype I32 : acc
 * out_dtype F32 : clamp((float)acc * (sx * sw), lo, hi)
 * out_dtype U8  : sat_u8(rne(clamp((float)acc * (sx*sw), lo, hi) / sy + (float)zy))
 * Padding taps contribute nothing.  This is the integer-exact form of what
 * nncase imports a quantized conv as -- Dequantize -> Conv2D(fused_clamp) ->
 * Quantize (src/Nncase.Importer/Onnx/QLinearConv.cs:61-75,
 * src/Nncase.Importer/TFLite/Conv2D.cs:39-98) -- and replaces
 * kernels::stackvm::conv2d (tensor_ops.cpp:181-220 ->
 * reference/convolution.cpp:26-105) on that sub-graph.  groups == 1 runs on
 * int8 MFMA, groups == in_channels == out_channels runs the depthwise
 * streaming kernel, other group counts run one MFMA launch per group.
 */
typedef struct nncase_hip_conv2d_desc {
    int32_t in_channels, out_channels;
    int32_t kernel_h, kernel_w;
    int32_t groups;
    nncase_hip_quant_param_t w_qp; /* per-tensor weight quantisation */
    /* batch * out_h * out_w the weights will be run with (shapes are static in a
     * kmodel); used only to pick a tiling that fills the device. 0 = unknown. */
    int64_t expected_pixels;
} nncase_hip_conv2d_desc_t;

/* Re-lays-out HOST weights (OIHW u8) and bias (int32[out_channels], may be
 * NULL = zeros) into the MFMA operand order, re-biases them to s8, computes
 * the per-output-channel sums used for zero-point correction and uploads the
 * result.  Done once per constant, like nncase's .rdata constants. */
NNCASE_HIP_API int nncase_hip_qconv2d_prepack(nncase_hip_ctx_t *ctx, const nncase_hip_conv2d_desc_t *desc,
                                              const uint8_t *weights_oihw_host, const int32_t *bias_host,
                                              nncase_hip_weights_t **weights);
NNCASE_HIP_API int nncase_hip_weights_destroy(nncase_hip_ctx_t *ctx, nncase_hip_weights_t *weights);
/* Attaches a fused unary operator to pre-packed dense (non-depthwise) weights:
 * a 256-entry host table (nncase_hip_make_unary_lut) that every u8-output call applies to the
 * requantised byte,  y = table[Q_y(conv)]  = Quantize(unary(Dequantize(conv result))) of the
 * u8/u8 graph, before the residual add if the call has one; table_qp is the quant param of the
 * table's output (the residual stage dequantises with it).  The activation that follows a
 * convolution is as static as its weights, so it is uploaded once with them.  NULL detaches. */
NNCASE_HIP_API int nncase_hip_weights_set_post_lut(nncase_hip_ctx_t *ctx, nncase_hip_weights_t *weights,
                                                   const uint8_t *lut256_host, nncase_hip_quant_param_t table_qp);

typedef struct nncase_hip_conv2d_args {
    int32_t batch, in_h, in_w;           /* input is [batch, in_h, in_w, in_channels] u8   */
    int32_t stride_h, stride_w;
    int32_t dilation_h, dilation_w;
    int32_t pad_h_before, pad_h_after;   /* paddings_t order of tensor_ops.cpp:192-199     */
    int32_t pad_w_before, pad_w_after;
    nncase_hip_quant_param_t x_qp;       /* input quantisation                             */
    nncase_hip_quant_param_t y_qp;       /* output quantisation (U8 output only)           */
    float clamp_min, clamp_max;          /* fused_clamp of Conv2D, applied in the fp32 domain */
    int32_t out_dtype;                   /* NNCASE_HIP_DT_U8 / _I32 / _F32                 */
    /* Optional fused residual add (U8 output, dense kernels only).  With residual_dev set
     * the call computes what nncase_hip_qconv2d followed by nncase_hip_qadd would:
     *   y = Q_sum(clamp(DQ_y(conv result requantised with y_qp) + DQ_res(residual)))
     * without writing the convolution's own u8 tensor.  residual_dev has the output's shape. */
    const uint8_t *residual_dev;
    nncase_hip_quant_param_t residual_qp;
    nncase_hip_quant_param_t sum_qp;
    float sum_clamp_min, sum_clamp_max;
    /* Output placed inside a wider NHWC tensor (the producer of one input of a channel concat writes
     * its slice of the concat's tensor): pixel stride in channels, 0 = out_channels (dense), and the
     * first channel written.  Dense (MFMA) kernels only; residual_dev stays a dense tensor. */
    int32_t out_channel_stride, out_channel_offset;
    /* With out_dtype == NNCASE_HIP_DT_F32 and dequantize_output != 0 the call computes the u8 result described
     * above (y_qp, the fused table and residual included) and stores its float32 value
     * (q - zero_point) * scale of the last stage's quant param instead of the byte: the Dequantize that
     * follows the last convolution of a quantised graph, bit-identical to nncase_hip_qconv2d followed by
     * nncase_hip_dequantize without the u8 tensor in between.  Dense (MFMA) kernels only, no out_channel_stride. */
    int32_t dequantize_output;
    int32_t reserved;                    /* 0 */
} nncase_hip_conv2d_args_t;

/* Output is [batch, out_h, out_w, out_channels] with
 * out = (in + pad_before + pad_after - ((k-1)*dilation+1) + stride) / stride
 * (src/Native/include/nncase/kernels/kernel_utils.h:86-93). */
NNCASE_HIP_API int nncase_hip_qconv2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_weights_t *weights,
                                      void *y_dev, const nncase_hip_conv2d_args_t *args);

/* Host-only view of the u8 requantisation  q = sat_u8(rne(clamp((float)acc * (sx * sw), lo, hi) / sy + zy))
 * (quantize.cpp:36-43 applied to Conv2D's clamped fp32 value, convolution.cpp:99-101) that the u8 epilogues run.
 * It is a monotone step function of the accumulator; where constants exist for which
 * RN(fma((float)acc, c1, c2)) steps at exactly the same accumulators, the kernels use that one
 * instruction instead of the three-rounding sequence.  nncase_hip_requant_plan returns 1 and the
 * constants if the search (every step of the staircase is compared) found a pair, else 0;
 * nncase_hip_requant_host evaluates the form the kernels would pick (form_used: 1 = fma form,
 * 0 = exact sequence) on host accumulators, so that callers and tests can compare it with their
 * own arithmetic.  Neither needs a device. */
NNCASE_HIP_API int nncase_hip_requant_plan(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                           float *c1, float *c2);
NNCASE_HIP_API int nncase_hip_requant_host(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                           const int32_t *acc_host, size_t count, uint8_t *out_host, int32_t *form_used);
/* The same for the form without an int -> float conversion that the dense row / window kernels and the stride-2
 * depthwise kernel use where it exists: the sums are started from 0x4B400000, so that their bits read as a float
 * are 12582912 + acc, and the code is RN(fma(that float, m1, m2)).  Returns 1 and writes the codes of the
 * accumulators (each of magnitude at most *limit, the range the search vouches for; others get 0) when the
 * search found a pair, 0 when it did not (nothing is written then), a negative status for scales out of range.
 * Host-only like the two above (no counterpart in the reference: its CPU kernel divides, quantize.cpp:36-43). */
NNCASE_HIP_API int nncase_hip_requant_host_magic(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                                 const int32_t *acc_host, size_t count, uint8_t *out_host, float *m1, float *m2,
                                                 int32_t *limit);

/* ---- fused inverted-residual block ------------------------------------------
 * 1x1 convolution (in -> mid channels), 3x3 depthwise convolution on the mid
 * channels (stride 1 or 2), 1x1 convolution (mid -> out channels), optionally
 * + the block's input: what the reference keeps as one Fusion function
 * (src/Nncase.Core/IR/Fusion.cs:13) of three Conv2D calls
 * (src/Native/src/kernels/stackvm/reference/convolution.cpp:26-143) and a
 * Binary add.  One kernel computes all of it per output tile: the two mid
 * tensors (the largest of the block) live in LDS only and never reach HBM.
 * The result is bit-identical to nncase_hip_qconv2d called three times (the
 * last with the input as fused residual) with the same quant params: every
 * stage requantises to u8 exactly as the separate operators do.
 */
typedef struct nncase_hip_qblock_weights nncase_hip_qblock_t;

typedef struct nncase_hip_qblock_desc {
    int32_t in_channels, mid_channels, out_channels;
    nncase_hip_quant_param_t expand_w_qp, dw_w_qp, project_w_qp; /* per-tensor weight quantisation of the stages */
} nncase_hip_qblock_desc_t;

/* 1 if the fused kernel is built for these channel counts (in_channels % 4 == 0 and <= 192,
 * mid_channels % 4 == 0, out_channels <= 320), else 0: the caller then runs the three convolutions. */
NNCASE_HIP_API int nncase_hip_qblock_supported(const nncase_hip_qblock_desc_t *desc);
/* HOST weights, OIHW u8: expand [mid, in, 1, 1], depthwise [mid, 1, 3, 3], project [out, mid, 1, 1];
 * int32 biases (NULL = zeros) in the accumulator scale of their stage. */
NNCASE_HIP_API int nncase_hip_qblock_prepack(nncase_hip_ctx_t *ctx, const nncase_hip_qblock_desc_t *desc,
                                             const uint8_t *w_expand_host, const int32_t *bias_expand_host,
                                             const uint8_t *w_dw_host, const int32_t *bias_dw_host,
                                             const uint8_t *w_project_host, const int32_t *bias_project_host,
                                             nncase_hip_qblock_t **block);
NNCASE_HIP_API int nncase_hip_qblock_destroy(nncase_hip_ctx_t *ctx, nncase_hip_qblock_t *block);

typedef struct nncase_hip_qblock_args {
    int32_t batch, in_h, in_w;           /* input is [batch, in_h, in_w, in_channels] u8            */
    int32_t stride;                      /* of the depthwise stage, both axes: 1 or 2               */
    int32_t pad_h_before, pad_h_after;   /* of the depthwise stage, each 0 or 1                     */
    int32_t pad_w_before, pad_w_after;
    nncase_hip_quant_param_t x_qp;       /* block input                                             */
    nncase_hip_quant_param_t expand_qp;  /* output of the 1x1 expansion                             */
    nncase_hip_quant_param_t dw_qp;      /* output of the depthwise stage                           */
    nncase_hip_quant_param_t y_qp;       /* output of the 1x1 projection                            */
    float expand_clamp_min, expand_clamp_max; /* fused_clamp of each stage, fp32 domain             */
    float dw_clamp_min, dw_clamp_max;
    float clamp_min, clamp_max;
    /* add_input != 0: y = Q_sum(clamp(DQ_y(projection) + DQ_x(x))), the residual connection
     * (needs stride 1 and out_channels == in_channels). */
    int32_t add_input;
    nncase_hip_quant_param_t sum_qp;
    float sum_clamp_min, sum_clamp_max;
} nncase_hip_qblock_args_t;

/* Output is [batch, out_h, out_w, out_channels] u8 with out = (in + pad_before + pad_after - 3 + stride) / stride. */
NNCASE_HIP_API int nncase_hip_qblock(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_qblock_t *block,
                                     uint8_t *y_dev, const nncase_hip_qblock_args_t *args);

/* Global average pool (ReduceMean over H and W of a u8 tensor, src/Native/src/kernels/stackvm/reference/reduce.cpp,
 * requantised to args->x_qp) and the dense 1x1 Conv2D that reads its [batch, 1, 1, channels] result as one launch: a
 * classifier's pool -> fully-connected tail at small batches.  x_dev is the pool's input [batch, h, w, channels] with
 * quantisation x_qp; args are the convolution's (in_h = in_w = 1; u8 output or dequantize_output).  Same bytes as
 * nncase_hip_qglobal_avgpool followed by nncase_hip_qconv2d.  The weights must have been pre-packed with
 * expected_pixels = the batch (a few rows): _supported says whether a call qualifies and pays (every workgroup pools
 * its rows itself, so only while rows x pixels x channels is small). */
NNCASE_HIP_API int nncase_hip_qglobal_avgpool_qconv2d_supported(const nncase_hip_weights_t *weights,
                                                                const nncase_hip_conv2d_args_t *args, int32_t h, int32_t w);
NNCASE_HIP_API int nncase_hip_qglobal_avgpool_qconv2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, int32_t h, int32_t w,
                                                      nncase_hip_quant_param_t x_qp, const nncase_hip_weights_t *weights,
                                                      void *y_dev, const nncase_hip_conv2d_args_t *args);

/* ---- pair of pointwise convolutions ------------------------------------------
 * Two dense 1x1, stride-1, unpadded Conv2D calls of which the second reads the
 * first's result (a bottleneck's projection and the next block's expansion,
 * which the importer leaves as separate Conv2D calls,
 * src/Nncase.Importer/TFLite/Conv2D.cs:17-69, each running
 * src/Native/src/kernels/stackvm/reference/convolution.cpp:26-143) as one launch:
 *   y1 = first(x)  [byte table of the first weights]  [+ first_args->residual_dev]
 *   y2 = second(y1) [byte table of the second weights]
 * Both results are stored; every byte equals what nncase_hip_qconv2d writes for
 * the two calls with the same arguments.  Meant for small pixel counts (batch 1,
 * late feature maps) where the two calls are bound by launch latency: each
 * workgroup recomputes the first convolution for its 16 pixels, so on large
 * tensors the two separate calls are faster.
 * The pair keeps pointers to both weights handles (bias, zero points, scales,
 * tables): they must outlive it.  The raw OIHW weights are needed again because
 * the pair packs them in its own order.
 * supported: in_channels a multiple of 16 up to 1024, mid_channels a multiple of
 * 4 up to 512, out_channels a multiple of 4. */
typedef struct nncase_hip_qpair nncase_hip_qpair_t;
NNCASE_HIP_API int nncase_hip_qpointwise_pair_supported(int32_t in_channels, int32_t mid_channels, int32_t out_channels);
NNCASE_HIP_API int nncase_hip_qpointwise_pair_create(nncase_hip_ctx_t *ctx, const nncase_hip_weights_t *first,
                                                     const uint8_t *first_oihw_host, const nncase_hip_weights_t *second,
                                                     const uint8_t *second_oihw_host, nncase_hip_qpair_t **pair);
NNCASE_HIP_API int nncase_hip_qpointwise_pair_destroy(nncase_hip_ctx_t *ctx, nncase_hip_qpair_t *pair);
/* first_args / second_args as for nncase_hip_qconv2d (u8 results, dense outputs; only the first may carry a residual);
 * second_args->x_qp is the quantisation of y1 as the second convolution reads it. */
NNCASE_HIP_API int nncase_hip_qpointwise_pair(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_qpair_t *pair,
                                              uint8_t *y1_dev, uint8_t *y2_dev, const nncase_hip_conv2d_args_t *first_args,
                                              const nncase_hip_conv2d_args_t *second_args);

/* The same with the 3x3 depthwise Conv2D (stride 1 or 2, no dilation) that produces x in front, still one launch:
 * x_dev is the DEPTHWISE convolution's input [batch, in_h, in_w, in_channels]; its result, which nothing else may
 * need, is never stored (each workgroup computes its 16 pixels of it into LDS).  depthwise is the prepack handle of
 * the depthwise weights (no table), depthwise_args its nncase_hip_qconv2d arguments; its y_qp must be first_args->x_qp
 * and its output extents first_args' input extents.  y1 and y2 are bit-identical to the three nncase_hip_qconv2d
 * calls. */
NNCASE_HIP_API int nncase_hip_qdepthwise_pointwise_pair(nncase_hip_ctx_t *ctx, const uint8_t *x_dev,
                                                        const nncase_hip_weights_t *depthwise,
                                                        const nncase_hip_conv2d_args_t *depthwise_args,
                                                        const nncase_hip_qpair_t *pair, uint8_t *y1_dev, uint8_t *y2_dev,
                                                        const nncase_hip_conv2d_args_t *first_args,
                                                        const nncase_hip_conv2d_args_t *second_args);

/* MatMul A[M,K] (u8, device) x B[K,N] (u8, row-major, HOST, pre-packed) with
 * the same three output forms; replaces kernels::stackvm::mat_mul
 * (tensor_ops.cpp:553-565 -> reference/matmul.cpp:28-48) on the
 * Dequantize -> MatMul (-> Quantize) sub-graph of
 * src/Nncase.Importer/Onnx/QLinearMatmul.cs:25-28. */
NNCASE_HIP_API int nncase_hip_qmatmul_prepack(nncase_hip_ctx_t *ctx, const uint8_t *b_host, int32_t k, int32_t n,
                                              nncase_hip_quant_param_t b_qp, const int32_t *bias_host,
                                              int64_t expected_rows, nncase_hip_weights_t **weights);

typedef struct nncase_hip_matmul_args {
    int32_t m;
    nncase_hip_quant_param_t a_qp;
    nncase_hip_quant_param_t y_qp;
    float clamp_min, clamp_max;
    int32_t out_dtype;
} nncase_hip_matmul_args_t;

NNCASE_HIP_API int nncase_hip_qmatmul(nncase_hip_ctx_t *ctx, const uint8_t *a_dev, const nncase_hip_weights_t *weights,
                                      void *y_dev, const nncase_hip_matmul_args_t *args);

/* ---- u8 glue that keeps a quantized graph resident --------------------- */

/* out = Q(clamp(DQ(a) + DQ(b))), elementwise on `count` bytes (binary add,
 * src/Native/src/kernels/stackvm/reference/binary.cpp, between the
 * dequantize / quantize formulas above). */
NNCASE_HIP_API int nncase_hip_qadd(nncase_hip_ctx_t *ctx, const uint8_t *a_dev, nncase_hip_quant_param_t a_qp,
                                   const uint8_t *b_dev, nncase_hip_quant_param_t b_qp, uint8_t *out_dev,
                                   nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max, size_t count);

/* out[n, c] = Q(mean_{h,w} DQ(x[n, h, w, c])): the sequential float window sum
 * of reduce_window2d mean (reference/reduce_window.cpp:36-109,133-135) over
 * the whole image. */
NNCASE_HIP_API int nncase_hip_qglobal_avgpool(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, uint8_t *out_dev,
                                              int32_t batch, int32_t h, int32_t w, int32_t channels,
                                              nncase_hip_quant_param_t x_qp, nncase_hip_quant_param_t y_qp);

/* u8 -> u8 operators between Dequantize and Quantize as 256-entry byte tables:
 * table[v] = Q_y(f(DQ_x(v))), evaluated on the host with the CPU kernels' fp32
 * operations (dequantize.cpp:36-39, quantize.cpp:36-43).
 *   NNCASE_HIP_LUT_REQUANT  f(x) = x: the Quantize(Dequantize(.)) pair a graph
 *                           holds where tensors of different quant params meet
 *   NNCASE_HIP_LUT_SWISH    f(x) = x / (1 + exp(-x)), unary swish
 *                           (src/Native/src/kernels/stackvm/reference/activation.cpp:36)
 * nncase_hip_make_unary_lut is host-only; nncase_hip_lut_u8 applies a table to
 * `count` bytes on the device. */
#define NNCASE_HIP_LUT_REQUANT 0
#define NNCASE_HIP_LUT_SWISH 1
NNCASE_HIP_API int nncase_hip_make_unary_lut(int32_t kind, nncase_hip_quant_param_t x_qp, nncase_hip_quant_param_t y_qp,
                                             uint8_t *lut256_host);
NNCASE_HIP_API int nncase_hip_lut_u8(nncase_hip_ctx_t *ctx, const uint8_t *in_dev, uint8_t *out_dev, size_t count,
                                     const uint8_t *lut256_host);

/* Concat along the channel axis of NHWC u8 tensors (kernels::stackvm::concat,
 * src/Native/src/kernels/stackvm/tensor_ops.cpp, on the innermost axis) with
 * every input requantised to the output's quant params, i.e. the
 * Dequantize -> Concat -> Quantize sub-graph of a u8/u8 model:
 *   out[p, off_i + c] = Q_out(DQ_i(in_i[p, c])),  off_i = channels_0 + .. + channels_{i-1}.
 * An input whose pointer is NULL is skipped: its channels are already in place (written there by
 * a convolution with out_channel_stride / out_channel_offset). */
#define NNCASE_HIP_MAX_CONCAT 8
NNCASE_HIP_API int nncase_hip_qconcat_channels(nncase_hip_ctx_t *ctx, int32_t n_inputs, const uint8_t *const *in_dev,
                                               const int32_t *channels, const nncase_hip_quant_param_t *in_qps,
                                               uint8_t *out_dev, nncase_hip_quant_param_t out_qp, int64_t pixels);

/* resize_image(nearest_neighbor) on an NHWC tensor of 1/2/4-byte elements
 * (kernels::stackvm::resize_image, tensor_ops.cpp:888-932;
 * reference/resize_image.cpp:91-139).  Mode values are the reference's
 * image_resize_transformation_mode_t / image_resize_nearest_mode_t
 * (src/Native/include/nncase/runtime/stackvm/opcode.h:330-343). */
#define NNCASE_HIP_RESIZE_HALF_PIXEL 0
#define NNCASE_HIP_RESIZE_PYTORCH_HALF_PIXEL 1
#define NNCASE_HIP_RESIZE_ALIGN_CORNERS 2
#define NNCASE_HIP_RESIZE_ASYMMETRIC 3
#define NNCASE_HIP_RESIZE_TFCROP_AND_RESIZE 4
#define NNCASE_HIP_NEAREST_ROUND_PREFER_FLOOR 0
#define NNCASE_HIP_NEAREST_ROUND_PREFER_CEIL 1
#define NNCASE_HIP_NEAREST_FLOOR 2
#define NNCASE_HIP_NEAREST_CEIL 3
NNCASE_HIP_API int nncase_hip_resize_nearest(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size,
                                             int32_t batch, int32_t in_h, int32_t in_w, int32_t channels, int32_t out_h,
                                             int32_t out_w, int32_t transformation_mode, int32_t nearest_mode);

/* reduce_window2d(max) between Dequantize and Quantize on NHWC u8
 * (kernels::stackvm::reduce_window2d, src/Native/src/kernels/stackvm/reference/reduce_window.cpp:35-109):
 *   out = Q_y(max over the window of DQ_x(x)), and, as in the reference's loop (:88-91), the value
 * 0 takes part once for every window position that lies in the padding.  Dilation 1. */
NNCASE_HIP_API int nncase_hip_qmaxpool2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, uint8_t *out_dev, int32_t batch,
                                         int32_t in_h, int32_t in_w, int32_t channels, int32_t kernel_h, int32_t kernel_w,
                                         int32_t stride_h, int32_t stride_w, int32_t pad_h_before, int32_t pad_h_after,
                                         int32_t pad_w_before, int32_t pad_w_after, nncase_hip_quant_param_t x_qp,
                                         nncase_hip_quant_param_t y_qp);

/* ---- pack / unpack ------------------------------------------------------
 * pack: every listed axis a (extent D) becomes an outer axis of extent
 * ceil(D / lanes) in place and its lane index is appended as a trailing axis
 * of extent `lanes`, in the order the axes are listed; elements past D are
 * zero.  unpack is the inverse with a crop.  A dimension permutation with
 * padding; elem_size in {1, 2, 4}.  (No counterpart in this reference tree.)
 */
NNCASE_HIP_API int nncase_hip_pack(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size,
                                   int32_t rank, const int32_t *shape, int32_t n_axes, const int32_t *axes,
                                   const int32_t *lanes);
NNCASE_HIP_API int nncase_hip_unpack(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size,
                                     int32_t rank, const int32_t *unpacked_shape, int32_t n_axes,
                                     const int32_t *axes, const int32_t *lanes);
/* Quantize (float32 -> u8, as nncase_hip_quantize) followed by pack, in one pass over the input: what stands in
 * front of a stem convolution over RGB.  Two layouts: <= 4 innermost channels packed by (4) (RGB -> RGBX), and an
 * NHWC tensor with <= 4 channels and even H, W packed by (2, 2, 4) on (H, W, C), which turns every 2 x 2 block of
 * pixels into one 16-channel pixel of the half-size image (a stride-2 convolution with an even window then reads it
 * as a stride-1 convolution with half the window).  out_dev must be 16-byte aligned; -EINVAL for other arguments.
 * The result equals nncase_hip_quantize then nncase_hip_pack byte for byte. */
NNCASE_HIP_API int nncase_hip_quantize_pack(nncase_hip_ctx_t *ctx, const float *in_dev, uint8_t *out_dev, int32_t rank,
                                            const int32_t *shape, int32_t n_axes, const int32_t *axes,
                                            const int32_t *lanes, nncase_hip_quant_param_t qp);

/* NCHW <-> NHWC relayout of a dense tensor (the Transpose nncase inserts
 * around NHWC imports, src/Nncase.Importer/TFLite/Conv2D.cs:28-29,67). */
NNCASE_HIP_API int nncase_hip_nchw_to_nhwc(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev,
                                           int32_t elem_size, int32_t n, int32_t c, int32_t h, int32_t w);
NNCASE_HIP_API int nncase_hip_nhwc_to_nchw(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev,
                                           int32_t elem_size, int32_t n, int32_t c, int32_t h, int32_t w);

/* ---- paged-attention decode ---------------------------------------------
 * One query token per sequence against a block-paged fp16 KV cache:
 *   out[b, h, :] = softmax(scale * q[b, h, :] . K[b, kvh, 0..ctx_b)) . V[b, kvh, ...]
 * with kvh = h / (num_q_heads / num_kv_heads), fp32 scores and accumulation.
 *   q            [batch, num_q_heads, head_dim]                 f16
 *   k cache      [num_blocks, num_kv_heads, block_size, head_dim] f16
 *   v cache      [num_blocks, num_kv_heads, head_dim, block_size] f16 (d-major:
 *                a lane's matrix-core operand, 4 consecutive tokens of one d,
 *                is then one 8-byte load)
 *   block_table  [batch, max_blocks_per_seq] int32 (physical block ids)
 *   ctx_lens     [batch] int32
 *   out          [batch, num_q_heads, head_dim]                 f16 or f32
 * head_dim 64 or 128; block_size a multiple of 16; at most 16 query heads per
 * kv head; scale may have either sign.  Slots of a block past the context
 * length may hold anything.  (No counterpart in this reference tree.)
 */
typedef struct nncase_hip_paged_attn_args {
    int32_t batch, num_q_heads, num_kv_heads, head_dim;
    int32_t block_size, max_blocks_per_seq, num_blocks;
    float scale;
    int32_t out_dtype; /* NNCASE_HIP_DT_F16 or _F32 */
    /* added to every ctx_lens[b] (a decode step attends to the token it has just appended, before the
     * lengths are advanced at the end of the step: 1; otherwise 0) */
    int32_t ctx_len_offset;
} nncase_hip_paged_attn_args_t;

NNCASE_HIP_API int nncase_hip_paged_attention_decode(nncase_hip_ctx_t *ctx, const void *q_dev, const void *k_cache_dev,
                                                     const void *v_cache_dev, const int32_t *block_table_dev,
                                                     const int32_t *ctx_lens_dev, void *out_dev,
                                                     const nncase_hip_paged_attn_args_t *args);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The split
 * partials and completion counters that nncase_hip_paged_attention_decode keeps in a workspace owned by the
 * context live here in a static device array of the library (8 MiB of partials + 64 KiB of counters per GPU,
 * held until the process ends); the call allocates and frees nothing and issues no memset.  Geometries whose
 * partials (batch * num_q_heads * splits * (head_dim + 2) floats, splits = context capacity / tokens per
 * split) or counters (batch * num_kv_heads words) exceed that are refused with -ENOSPC.  All calls on one GPU
 * share the array: calls that overlap in time on one GPU (two contexts, two streams) race; calls on one
 * context are ordered by its stream.  Results are bit-identical to nncase_hip_paged_attention_decode. */
NNCASE_HIP_API int nncase_hip_paged_attention_decode_noalloc(nncase_hip_ctx_t *ctx, const void *q_dev, const void *k_cache_dev,
                                                             const void *v_cache_dev, const int32_t *block_table_dev,
                                                             const int32_t *ctx_lens_dev, void *out_dev,
                                                             const nncase_hip_paged_attn_args_t *args);

/* ---- the rest of an LLM decode step (fp16 activations, W8A16 weights) --------
 * No counterpart in this reference tree (its LLM path lives in another branch); the
 * arithmetic is defined here and checked against float64 restatements.
 *
 * W8A16 linear layer: out[m, n] = scale[n] * sum_k a[m, k] * w[n, k] (+ bias[n]), a fp16,
 * w int8 with one fp32 scale per output channel, fp32 accumulation.  k a multiple of 64,
 * n a multiple of 16, 1..64 token rows per call.
 *   NNCASE_HIP_GEMM_PLAIN   out is [m, n]
 *   NNCASE_HIP_GEMM_SWIGLU  the matrix holds the gate projection in rows [0, n/2) and the up
 *                           projection in rows [n/2, n): out[m, j] = silu(gate_j) * up_j, [m, n/2]
 * residual_dev (fp16, shape of out, 8-byte aligned, may be NULL) is added to the result; out is fp16 or fp32
 * (a_dev and out_dev 16-byte aligned; -invalid_memory_location otherwise). */
#define NNCASE_HIP_GEMM_PLAIN 0
#define NNCASE_HIP_GEMM_SWIGLU 1
typedef struct nncase_hip_w8a16 nncase_hip_w8a16_t;
NNCASE_HIP_API int nncase_hip_w8a16_prepack(nncase_hip_ctx_t *ctx, const int8_t *w_nk_host, const float *scale_host,
                                            const float *bias_host, int32_t k, int32_t n, nncase_hip_w8a16_t **weights);
NNCASE_HIP_API int nncase_hip_w8a16_destroy(nncase_hip_ctx_t *ctx, nncase_hip_w8a16_t *weights);
NNCASE_HIP_API int nncase_hip_w8a16_gemm(nncase_hip_ctx_t *ctx, const void *a_dev, const nncase_hip_w8a16_t *weights,
                                         void *out_dev, int32_t m, int32_t mode, const void *residual_dev, int32_t out_dtype);
/* The same product on rmsnorm(x) (below) without the normalised rows passing through memory: bit for bit what
 * nncase_hip_rmsnorm_f16 followed by nncase_hip_w8a16_gemm writes.  ln_weight_dev: [k] fp16, 16-byte aligned. */
NNCASE_HIP_API int nncase_hip_rmsnorm_w8a16_gemm(nncase_hip_ctx_t *ctx, const void *x_dev, const void *ln_weight_dev, float eps,
                                                 const nncase_hip_w8a16_t *weights, void *out_dev, int32_t m, int32_t mode,
                                                 const void *residual_dev, int32_t out_dtype);
/* out[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight, fp16 in / out, fp32 arithmetic. */
NNCASE_HIP_API int nncase_hip_rmsnorm_f16(nncase_hip_ctx_t *ctx, const void *x_dev, const void *weight_dev, void *out_dev,
                                          int32_t rows, int32_t hidden, float eps);
/* qkv [batch, (Hq + 2 Hkv) * d] fp16 (q heads, k heads, v heads) of one new token per sequence:
 * rotary embedding (rotate-half pairing, angle pos * theta^(-2i/d), pos = ctx_lens[b]) of q and k;
 * q goes to q_out [batch, Hq, d], the rotated k and v are appended at position ctx_lens[b] of the
 * paged cache (layouts of nncase_hip_paged_attention_decode).  ctx_lens is NOT advanced. */
NNCASE_HIP_API int nncase_hip_rope_kv_append(nncase_hip_ctx_t *ctx, const void *qkv_dev, void *q_out_dev, void *k_cache_dev,
                                             void *v_cache_dev, const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                             const nncase_hip_paged_attn_args_t *geometry, float rope_theta);
/* The q / k / v projection of (optionally RMS-normalised, ln_weight_dev may be null) rows x, followed by
 * nncase_hip_rope_kv_append, as one launch where the geometry allows (up to 32 rows, head_dim a multiple of 32, a
 * reduction of up to 1024): the block that multiplies a tile of a head also multiplies the tile half a head further,
 * so the rotate-half pairs meet in its epilogue.  The values are those of nncase_hip_rmsnorm_w8a16_gemm (or
 * nncase_hip_w8a16_gemm) into fp16 followed by nncase_hip_rope_kv_append, bit for bit; qkv_dev [batch, (Hq + 2 Hkv) * d]
 * is scratch that the two-launch form of other geometries writes. */
NNCASE_HIP_API int nncase_hip_w8a16_gemm_rope_kv_append(nncase_hip_ctx_t *ctx, const void *x_dev, const void *ln_weight_dev,
                                                        float eps, const nncase_hip_w8a16_t *weights, void *qkv_dev,
                                                        void *q_out_dev, void *k_cache_dev, void *v_cache_dev,
                                                        const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                                        const nncase_hip_paged_attn_args_t *geometry, float rope_theta);
/* out[r] = index of the largest element of row r (the lowest index among equals). */
NNCASE_HIP_API int nncase_hip_argmax_f32(nncase_hip_ctx_t *ctx, const float *x_dev, int32_t *out_dev, int32_t rows, int32_t cols);
/* out[r, :] = table[ids[r], :] (fp16 rows). */
NNCASE_HIP_API int nncase_hip_embedding_f16(nncase_hip_ctx_t *ctx, const void *table_dev, const int32_t *ids_dev, void *out_dev,
                                            int32_t rows, int32_t hidden, int32_t vocab);
/* x[i] += delta (advances the context lengths after a decode step). */
NNCASE_HIP_API int nncase_hip_add_i32(nncase_hip_ctx_t *ctx, int32_t *x_dev, int32_t count, int32_t delta);

/* ---- resident functions --------------------------------------------------
 * A function is the `hip` module's counterpart of a runtime_function
 * (src/Native/include/nncase/runtime/runtime_function.h:55-63): an ordered
 * list of the operators above with their device operands bound, built once
 * when the module is loaded and invoked many times.  invoke() enqueues every
 * operator on the context's stream in order and returns; after
 * nncase_hip_function_capture() the same sequence is replayed as one HIP
 * graph launch (the operands must stay where they were when captured).
 * Operand buffers and weights stay owned by the caller and must outlive the
 * function.
 */
typedef struct nncase_hip_function nncase_hip_function_t;

NNCASE_HIP_API int nncase_hip_function_create(nncase_hip_ctx_t *ctx, nncase_hip_function_t **fn);
NNCASE_HIP_API int nncase_hip_function_destroy(nncase_hip_function_t *fn);
NNCASE_HIP_API int nncase_hip_function_add_quantize(nncase_hip_function_t *fn, const void *in_dev, int in_dtype,
                                                    void *out_dev, int out_dtype, size_t count,
                                                    nncase_hip_quant_param_t qp);
NNCASE_HIP_API int nncase_hip_function_add_dequantize(nncase_hip_function_t *fn, const void *in_dev, int in_dtype,
                                                      void *out_dev, int out_dtype, size_t count,
                                                      nncase_hip_quant_param_t qp);
NNCASE_HIP_API int nncase_hip_function_add_qconv2d(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                   const nncase_hip_weights_t *weights, void *y_dev,
                                                   const nncase_hip_conv2d_args_t *args);
NNCASE_HIP_API int nncase_hip_function_add_qblock(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                  const nncase_hip_qblock_t *block, uint8_t *y_dev,
                                                  const nncase_hip_qblock_args_t *args);
NNCASE_HIP_API int nncase_hip_function_add_qpointwise_pair(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                           const nncase_hip_qpair_t *pair, uint8_t *y1_dev, uint8_t *y2_dev,
                                                           const nncase_hip_conv2d_args_t *first_args,
                                                           const nncase_hip_conv2d_args_t *second_args);
NNCASE_HIP_API int nncase_hip_function_add_qdepthwise_pointwise_pair(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                                     const nncase_hip_weights_t *depthwise,
                                                                     const nncase_hip_conv2d_args_t *depthwise_args,
                                                                     const nncase_hip_qpair_t *pair, uint8_t *y1_dev,
                                                                     uint8_t *y2_dev,
                                                                     const nncase_hip_conv2d_args_t *first_args,
                                                                     const nncase_hip_conv2d_args_t *second_args);
NNCASE_HIP_API int nncase_hip_function_add_qglobal_avgpool_qconv2d(nncase_hip_function_t *fn, const uint8_t *x_dev, int32_t h,
                                                                   int32_t w, nncase_hip_quant_param_t x_qp,
                                                                   const nncase_hip_weights_t *weights, void *y_dev,
                                                                   const nncase_hip_conv2d_args_t *args);
NNCASE_HIP_API int nncase_hip_function_add_qadd(nncase_hip_function_t *fn, const uint8_t *a_dev,
                                                nncase_hip_quant_param_t a_qp, const uint8_t *b_dev,
                                                nncase_hip_quant_param_t b_qp, uint8_t *out_dev,
                                                nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                                size_t count);
NNCASE_HIP_API int nncase_hip_function_add_qglobal_avgpool(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                           uint8_t *out_dev, int32_t batch, int32_t h, int32_t w,
                                                           int32_t channels, nncase_hip_quant_param_t x_qp,
                                                           nncase_hip_quant_param_t y_qp);
NNCASE_HIP_API int nncase_hip_function_add_lut_u8(nncase_hip_function_t *fn, const uint8_t *in_dev, uint8_t *out_dev,
                                                  size_t count, const uint8_t *lut256_host);
NNCASE_HIP_API int nncase_hip_function_add_qconcat_channels(nncase_hip_function_t *fn, int32_t n_inputs,
                                                            const uint8_t *const *in_dev, const int32_t *channels,
                                                            const nncase_hip_quant_param_t *in_qps, uint8_t *out_dev,
                                                            nncase_hip_quant_param_t out_qp, int64_t pixels);
NNCASE_HIP_API int nncase_hip_function_add_resize_nearest(nncase_hip_function_t *fn, const void *in_dev, void *out_dev,
                                                          int32_t elem_size, int32_t batch, int32_t in_h, int32_t in_w,
                                                          int32_t channels, int32_t out_h, int32_t out_w,
                                                          int32_t transformation_mode, int32_t nearest_mode);
/* NCHW <-> NHWC relayout as a step of a function (nncase_hip_nchw_to_nhwc / nncase_hip_nhwc_to_nchw with the same
 * extents): the IR holds activations as NCHW, a hip function works channels-last, so a compiled function converts at
 * its two ends (the Transpose pair around NHWC imports, src/Nncase.Importer/TFLite/Conv2D.cs:28-29,67). */
NNCASE_HIP_API int nncase_hip_function_add_layout(nncase_hip_function_t *fn, const void *in_dev, void *out_dev,
                                                  int32_t elem_size, int32_t n, int32_t c, int32_t h, int32_t w,
                                                  int32_t to_nchw);
NNCASE_HIP_API int nncase_hip_function_add_qmaxpool2d(nncase_hip_function_t *fn, const uint8_t *x_dev, uint8_t *out_dev,
                                                      int32_t batch, int32_t in_h, int32_t in_w, int32_t channels,
                                                      int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
                                                      int32_t pad_h_before, int32_t pad_h_after, int32_t pad_w_before,
                                                      int32_t pad_w_after, nncase_hip_quant_param_t x_qp,
                                                      nncase_hip_quant_param_t y_qp);
/* pack with the arguments of nncase_hip_pack (rank <= 8); used e.g. to pad the channels of an RGB
 * tensor to 4 before its convolution. */
NNCASE_HIP_API int nncase_hip_function_add_pack(nncase_hip_function_t *fn, const void *in_dev, void *out_dev,
                                                int32_t elem_size, int32_t rank, const int32_t *shape, int32_t n_axes,
                                                const int32_t *axes, const int32_t *lanes);
NNCASE_HIP_API int nncase_hip_function_add_quantize_pack(nncase_hip_function_t *fn, const float *in_dev, uint8_t *out_dev,
                                                         int32_t rank, const int32_t *shape, int32_t n_axes,
                                                         const int32_t *axes, const int32_t *lanes,
                                                         nncase_hip_quant_param_t qp);
/* The decode-step operators above, recorded with the same arguments (paged attention included), so a
 * whole decode step replays as one HIP graph. */
NNCASE_HIP_API int nncase_hip_function_add_w8a16_gemm(nncase_hip_function_t *fn, const void *a_dev, const nncase_hip_w8a16_t *weights,
                                                      void *out_dev, int32_t m, int32_t mode, const void *residual_dev,
                                                      int32_t out_dtype);
NNCASE_HIP_API int nncase_hip_function_add_rmsnorm_w8a16_gemm(nncase_hip_function_t *fn, const void *x_dev,
                                                              const void *ln_weight_dev, float eps,
                                                              const nncase_hip_w8a16_t *weights, void *out_dev, int32_t m,
                                                              int32_t mode, const void *residual_dev, int32_t out_dtype);
NNCASE_HIP_API int nncase_hip_function_add_rmsnorm_f16(nncase_hip_function_t *fn, const void *x_dev, const void *weight_dev,
                                                       void *out_dev, int32_t rows, int32_t hidden, float eps);
NNCASE_HIP_API int nncase_hip_function_add_rope_kv_append(nncase_hip_function_t *fn, const void *qkv_dev, void *q_out_dev,
                                                          void *k_cache_dev, void *v_cache_dev, const int32_t *block_table_dev,
                                                          const int32_t *ctx_lens_dev,
                                                          const nncase_hip_paged_attn_args_t *geometry, float rope_theta);
NNCASE_HIP_API int nncase_hip_function_add_w8a16_gemm_rope_kv_append(nncase_hip_function_t *fn, const void *x_dev,
                                                                     const void *ln_weight_dev, float eps,
                                                                     const nncase_hip_w8a16_t *weights, void *qkv_dev,
                                                                     void *q_out_dev, void *k_cache_dev, void *v_cache_dev,
                                                                     const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                                                     const nncase_hip_paged_attn_args_t *geometry,
                                                                     float rope_theta);
NNCASE_HIP_API int nncase_hip_function_add_paged_attention_decode(nncase_hip_function_t *fn, const void *q_dev,
                                                                  const void *k_cache_dev, const void *v_cache_dev,
                                                                  const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                                                  void *out_dev, const nncase_hip_paged_attn_args_t *args);
NNCASE_HIP_API int nncase_hip_function_add_argmax_f32(nncase_hip_function_t *fn, const float *x_dev, int32_t *out_dev,
                                                      int32_t rows, int32_t cols);
NNCASE_HIP_API int nncase_hip_function_add_embedding_f16(nncase_hip_function_t *fn, const void *table_dev, const int32_t *ids_dev,
                                                         void *out_dev, int32_t rows, int32_t hidden, int32_t vocab);
NNCASE_HIP_API int nncase_hip_function_add_add_i32(nncase_hip_function_t *fn, int32_t *x_dev, int32_t count, int32_t delta);
/* Operators recorded after this call belong to independent chain `lane` (default 0).  Operators of one
 * lane run in the order recorded; different lanes must not touch each other's tensors.  A captured function
 * runs its lanes concurrently (e.g. the two halves of a batch, whose small layers cannot fill the device
 * alone); eager invocation runs all operators in the order recorded.  Paged attention and other operators
 * that use the context's scratch memory must stay in one lane.
 * NNCASE_HIP_LANE_JOINED: operators recorded after set_lane(fn, NNCASE_HIP_LANE_JOINED) wait for every lane and run as
 * one chain behind them (a step that ends in one product over the whole batch, whose weights the lanes would
 * otherwise each read); they have to be the last ones recorded. */
#define NNCASE_HIP_MAX_LANES 8
#define NNCASE_HIP_LANE_JOINED (-1)
NNCASE_HIP_API int nncase_hip_function_set_lane(nncase_hip_function_t *fn, int32_t lane);
/* Number of operators recorded so far. */
NNCASE_HIP_API int nncase_hip_function_size(nncase_hip_function_t *fn, int32_t *count);
/* Enqueues the whole function (graph replay if captured). */
NNCASE_HIP_API int nncase_hip_function_invoke(nncase_hip_function_t *fn);
/* Enqueues operator `index` alone (per-operator timing and debugging). */
NNCASE_HIP_API int nncase_hip_function_invoke_one(nncase_hip_function_t *fn, int32_t index);
/* Captures the operator sequence into a HIP graph used by later invokes. */
NNCASE_HIP_API int nncase_hip_function_capture(nncase_hip_function_t *fn);
/* Per-operator device time: every operator is enqueued `iterations` times
 * back to back between two HIP events recorded on the context's stream and
 * the mean duration in milliseconds is written to avg_ms[index] (the array
 * holds nncase_hip_function_size entries).  Blocks until done.  The HIP
 * counterpart of the reference's per-op profiler
 * (src/Native/include/nncase/runtime/stackvm/op_profile.h:41-76). */
NNCASE_HIP_API int nncase_hip_function_profile(nncase_hip_function_t *fn, int32_t iterations, float *avg_ms);
/* Name of the kernel operator `index` launches, e.g.
 * "qconv_igemm<T=9,RG=2,rows16>"; NUL-terminated, truncated to `capacity`. */
NNCASE_HIP_API int nncase_hip_function_op_kernel(nncase_hip_function_t *fn, int32_t index, char *name,
                                                 size_t capacity);

/* ---- kmodel v7 files with a "hip" entry module -------------------------------
 * Loads a kmodel (container of src/Native/include/nncase/runtime/model.h:38-74,
 * validated like interpreter::initialize_model, src/Native/src/runtime/
 * interpreter.cpp:95-102) whose entry function lives in a module of kind
 * "hip": uploads and pre-packs the module's .rdata constants, allocates one
 * device buffer per tensor and records the function's operator list into a
 * resident function (residual adds are folded into the dense convolution that
 * feeds them).  This is what the hip runtime module's initialize_before_functions
 * / runtime_function::initialize_core do
 * (src/Native/include/nncase/runtime/runtime_module.h, runtime_function.h:55-63).
 * The file image may be released after the call. */
typedef struct nncase_hip_kmodel nncase_hip_kmodel_t;
NNCASE_HIP_API int nncase_hip_kmodel_load(nncase_hip_ctx_t *ctx, const void *data, size_t size, nncase_hip_kmodel_t **kmodel);
/* The same for ONE function of a hip module, from the two byte ranges the reference's
 * runtime gives a runtime_function: `text` is the function's slice of the module's .text
 * section (function_header::entrypoint / text_size, model.h:60-67), `rdata` the module's
 * .rdata section (may be empty).  This is the call a hip runtime_function's
 * initialize_core makes (the stackvm counterpart takes the same two spans:
 * src/Native/src/runtime/stackvm/runtime_module.cpp:27-30, runtime_function.cpp:31-36). */
NNCASE_HIP_API int nncase_hip_kmodel_load_function(nncase_hip_ctx_t *ctx, const void *text, size_t text_size,
                                                   const void *rdata, size_t rdata_size, nncase_hip_kmodel_t **kmodel);
NNCASE_HIP_API int nncase_hip_kmodel_destroy(nncase_hip_kmodel_t *kmodel);
/* The entry function (owned by the kmodel): invoke / capture / profile it with nncase_hip_function_*. */
NNCASE_HIP_API int nncase_hip_kmodel_function(nncase_hip_kmodel_t *kmodel, nncase_hip_function_t **fn);
/* Device buffer, typecode and NHWC extents of the entry function's input / output
 * (interpreter::input_tensor / output_tensor) or of tensor `which` >= 0; the pointer is
 * NULL for a tensor that only exists inside a fused operator. */
#define NNCASE_HIP_KMODEL_INPUT (-1)
#define NNCASE_HIP_KMODEL_OUTPUT (-2) /* output k of a function with several outputs: NNCASE_HIP_KMODEL_OUTPUT - k */
NNCASE_HIP_API int nncase_hip_kmodel_tensor(nncase_hip_kmodel_t *kmodel, int32_t which, void **dev_ptr, int32_t *dtype,
                                            int32_t *dims4);

#ifdef __cplusplus
}
#endif
#endif /* NNCASE_HIP_H */
