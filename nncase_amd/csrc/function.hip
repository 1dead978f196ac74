// Resident functions: an ordered operator list bound to device operands,
// replayable eagerly or as one HIP graph.
#include "qconv.hpp"

#include <new>
#include <vector>

namespace {

struct Op {
    enum Kind { kQuantize, kDequantize, kConv, kAdd, kPool, kLut, kConcat, kResize, kMaxPool, kPack, kQuantPack,
                kGemm, kRmsNorm, kRope, kGemmRope, kAttn, kArgmax, kEmbed, kAddI32, kBlock, kLayout, kPair, kPoolConv } kind;
    const void *in0 = nullptr, *in1 = nullptr;
    void *out = nullptr;
    const nncase_hip_weights_t *weights = nullptr;
    nncase_hip_conv2d_args_t conv{};
    nncase_hip_quant_param_t qp0{}, qp1{}, qp2{};
    int dt_in = 0, dt_out = 0;
    size_t count = 0;
    float lo = 0.f, hi = 0.f;
    int32_t batch = 0, h = 0, w = 0, channels = 0;
    // byte table / concat / resize
    uint8_t lut[256] = {0};
    int32_t n_inputs = 0;
    const uint8_t *cat_in[NNCASE_HIP_MAX_CONCAT] = {nullptr};
    int32_t cat_channels[NNCASE_HIP_MAX_CONCAT] = {0};
    nncase_hip_quant_param_t cat_qp[NNCASE_HIP_MAX_CONCAT] = {};
    int64_t pixels = 0;
    int32_t elem_size = 0, out_h = 0, out_w = 0, tmode = 0, nmode = 0;
    int32_t pool[8] = {0}; // kernel h, w, stride h, w, pad h before / after, w before / after
    int32_t rank = 0, n_axes = 0, shape[8] = {0}, axes[8] = {0}, lanes[8] = {0};
    // decode-step operators
    const nncase_hip_w8a16_t *w8 = nullptr;
    const void *in2 = nullptr, *in3 = nullptr, *in4 = nullptr; // further operands (caches, tables)
    void *out2 = nullptr, *out3 = nullptr;
    nncase_hip_paged_attn_args_t attn{};
    int32_t mode = 0, delta = 0;
    float eps = 0.f, theta = 0.f;
    const nncase_hip_qblock_t *block = nullptr;
    nncase_hip_qblock_args_t blk{};
    // pair: conv (first) and conv2 (second) arguments, out / out2 the two results; with `weights` a depthwise
    // convolution in front, whose arguments are conv3
    const nncase_hip_qpair_t *pair = nullptr;
    nncase_hip_conv2d_args_t conv2{}, conv3{};
    int lane = 0; // independent operator chain this operator belongs to
};

} // namespace

struct nncase_hip_function {
    nncase_hip_ctx *ctx = nullptr;
    std::vector<Op> ops;
    int cur_lane = 0, nlanes = 1;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    bool pins_attn = false; // the captured graph holds the addresses of the context's attention workspace
    // Paged attention on a lane other than 0 goes through split partials and counters of that lane's own (lane 0
    // uses the context's), so that lanes may run it side by side; owned by the function.
    void *lane_partials[NNCASE_HIP_MAX_LANES] = {nullptr}, *lane_counters[NNCASE_HIP_MAX_LANES] = {nullptr};
    size_t lane_partial_bytes[NNCASE_HIP_MAX_LANES] = {0}, lane_counter_bytes[NNCASE_HIP_MAX_LANES] = {0};
};

using namespace nnhip;

static int run_op(nncase_hip_function *fn, const Op &op) {
    nncase_hip_ctx *ctx = fn->ctx;
    switch (op.kind) {
    case Op::kQuantize:
        return nncase_hip_quantize(ctx, op.in0, op.dt_in, op.out, op.dt_out, op.count, op.qp0);
    case Op::kDequantize:
        return nncase_hip_dequantize(ctx, op.in0, op.dt_in, op.out, op.dt_out, op.count, op.qp0);
    case Op::kConv:
        return nncase_hip_qconv2d(ctx, (const uint8_t *)op.in0, op.weights, op.out, &op.conv);
    case Op::kBlock:
        return nncase_hip_qblock(ctx, (const uint8_t *)op.in0, op.block, (uint8_t *)op.out, &op.blk);
    case Op::kPair:
        if (op.weights)
            return nncase_hip_qdepthwise_pointwise_pair(ctx, (const uint8_t *)op.in0, op.weights, &op.conv3, op.pair, (uint8_t *)op.out,
                                                        (uint8_t *)op.out2, &op.conv, &op.conv2);
        return nncase_hip_qpointwise_pair(ctx, (const uint8_t *)op.in0, op.pair, (uint8_t *)op.out, (uint8_t *)op.out2, &op.conv, &op.conv2);
    case Op::kPoolConv: // h, w and qp0 the pool's input, conv the convolution behind it
        return nncase_hip_qglobal_avgpool_qconv2d(ctx, (const uint8_t *)op.in0, op.h, op.w, op.qp0, op.weights, op.out, &op.conv);
    case Op::kAdd:
        return nncase_hip_qadd(ctx, (const uint8_t *)op.in0, op.qp0, (const uint8_t *)op.in1, op.qp1, (uint8_t *)op.out,
                               op.qp2, op.lo, op.hi, op.count);
    case Op::kPool:
        return nncase_hip_qglobal_avgpool(ctx, (const uint8_t *)op.in0, (uint8_t *)op.out, op.batch, op.h, op.w,
                                          op.channels, op.qp0, op.qp1);
    case Op::kLut:
        return nncase_hip_lut_u8(ctx, (const uint8_t *)op.in0, (uint8_t *)op.out, op.count, op.lut);
    case Op::kConcat:
        return nncase_hip_qconcat_channels(ctx, op.n_inputs, op.cat_in, op.cat_channels, op.cat_qp, (uint8_t *)op.out,
                                           op.qp0, op.pixels);
    case Op::kMaxPool:
        return nncase_hip_qmaxpool2d(ctx, (const uint8_t *)op.in0, (uint8_t *)op.out, op.batch, op.h, op.w, op.channels,
                                     op.pool[0], op.pool[1], op.pool[2], op.pool[3], op.pool[4], op.pool[5], op.pool[6],
                                     op.pool[7], op.qp0, op.qp1);
    case Op::kPack:
        return nncase_hip_pack(ctx, op.in0, op.out, op.elem_size, op.rank, op.shape, op.n_axes, op.axes, op.lanes);
    case Op::kQuantPack:
        return nncase_hip_quantize_pack(ctx, (const float *)op.in0, (uint8_t *)op.out, op.rank, op.shape, op.n_axes, op.axes, op.lanes, op.qp0);
    case Op::kGemm:
        if (op.in2) return nncase_hip_rmsnorm_w8a16_gemm(ctx, op.in0, op.in2, op.eps, op.w8, op.out, op.batch, op.mode, op.in1, op.dt_out);
        return nncase_hip_w8a16_gemm(ctx, op.in0, op.w8, op.out, op.batch, op.mode, op.in1, op.dt_out);
    case Op::kRmsNorm:
        return nncase_hip_rmsnorm_f16(ctx, op.in0, op.in1, op.out, op.batch, op.channels, op.eps);
    case Op::kGemmRope: // in0 rows, in1 normalisation weights, out the qkv scratch, out2 / out3 the caches, in2 block table, in3 lengths, in4 the query buffer
        return nncase_hip_w8a16_gemm_rope_kv_append(ctx, op.in0, op.in1, op.eps, op.w8, op.out, const_cast<void *>(op.in4), op.out2, op.out3,
                                                    (const int32_t *)op.in2, (const int32_t *)op.in3, &op.attn, op.theta);
    case Op::kRope:
        return nncase_hip_rope_kv_append(ctx, op.in0, op.out, op.out2, op.out3, (const int32_t *)op.in2, (const int32_t *)op.in3,
                                         &op.attn, op.eps);
    case Op::kAttn:
        if (op.lane > 0)
            return attn_decode_on(ctx, op.in0, op.in1, op.in2, (const int32_t *)op.in3, (const int32_t *)op.in4, op.out, &op.attn,
                                  fn->lane_partials[op.lane], fn->lane_partial_bytes[op.lane], fn->lane_counters[op.lane],
                                  fn->lane_counter_bytes[op.lane]);
        return nncase_hip_paged_attention_decode(ctx, op.in0, op.in1, op.in2, (const int32_t *)op.in3, (const int32_t *)op.in4,
                                                 op.out, &op.attn);
    case Op::kArgmax:
        return nncase_hip_argmax_f32(ctx, (const float *)op.in0, (int32_t *)op.out, op.batch, op.channels);
    case Op::kEmbed:
        return nncase_hip_embedding_f16(ctx, op.in0, (const int32_t *)op.in1, op.out, op.batch, op.channels, op.w);
    case Op::kAddI32:
        return nncase_hip_add_i32(ctx, (int32_t *)op.out, op.batch, op.delta);
    case Op::kLayout: // mode 0: NCHW -> NHWC, 1: NHWC -> NCHW
        return op.mode ? nncase_hip_nhwc_to_nchw(ctx, op.in0, op.out, op.elem_size, op.batch, op.channels, op.h, op.w)
                       : nncase_hip_nchw_to_nhwc(ctx, op.in0, op.out, op.elem_size, op.batch, op.channels, op.h, op.w);
    case Op::kResize:
        return nncase_hip_resize_nearest(ctx, op.in0, op.out, op.elem_size, op.batch, op.h, op.w, op.channels, op.out_h,
                                         op.out_w, op.tmode, op.nmode);
    }
    return -EINVAL;
}

static void drop_graph(nncase_hip_function *fn) {
    if (fn->exec) (void)hipGraphExecDestroy(fn->exec);
    if (fn->graph) (void)hipGraphDestroy(fn->graph);
    fn->exec = nullptr;
    fn->graph = nullptr;
    if (fn->pins_attn) fn->ctx->attn_pins--;
    fn->pins_attn = false;
}

static int push(nncase_hip_function *fn, const Op &op) {
    // (eager invocation runs the list in order: what waits for every lane has to come last)
    NNHIP_REQUIRE(fn->ctx, fn->cur_lane == NNCASE_HIP_LANE_JOINED || fn->ops.empty() || fn->ops.back().lane != NNCASE_HIP_LANE_JOINED, -EINVAL,
                  "function: operators behind the join of the lanes must be recorded last");
    drop_graph(fn); // a captured graph no longer matches the list
    fn->ops.push_back(op);
    fn->ops.back().lane = fn->cur_lane;
    return 0;
}

extern "C" int nncase_hip_function_set_lane(nncase_hip_function_t *fn, int32_t lane) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, lane == NNCASE_HIP_LANE_JOINED || (lane >= 0 && lane < NNCASE_HIP_MAX_LANES), -EINVAL,
                  "function_set_lane: lane %d (0..%d, or NNCASE_HIP_LANE_JOINED)", lane, NNCASE_HIP_MAX_LANES - 1);
    fn->cur_lane = lane;
    if (lane + 1 > fn->nlanes) fn->nlanes = lane + 1;
    return 0;
}

extern "C" int nncase_hip_function_create(nncase_hip_ctx_t *ctx, nncase_hip_function_t **out) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, out, -EINVAL, "function_create: null out pointer");
    nncase_hip_function *fn = new (std::nothrow) nncase_hip_function();
    NNHIP_REQUIRE(ctx, fn, -ENOMEM, "function_create: out of host memory");
    fn->ctx = ctx;
    *out = fn;
    return 0;
}

extern "C" int nncase_hip_function_destroy(nncase_hip_function_t *fn) {
    if (!fn) return -EINVAL;
    (void)hipStreamSynchronize(fn->ctx->stream);
    drop_graph(fn);
    for (int l = 0; l < NNCASE_HIP_MAX_LANES; l++) {
        if (fn->lane_partials[l]) (void)hipFree(fn->lane_partials[l]);
        if (fn->lane_counters[l]) (void)hipFree(fn->lane_counters[l]);
    }
    delete fn;
    return 0;
}

extern "C" int nncase_hip_function_add_quantize(nncase_hip_function_t *fn, const void *in_dev, int in_dtype, void *out_dev,
                                                int out_dtype, size_t count, nncase_hip_quant_param_t qp) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev, -EINVAL, "function_add_quantize: null buffer");
    Op op;
    op.kind = Op::kQuantize;
    op.in0 = in_dev, op.out = out_dev, op.dt_in = in_dtype, op.dt_out = out_dtype, op.count = count, op.qp0 = qp;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_dequantize(nncase_hip_function_t *fn, const void *in_dev, int in_dtype, void *out_dev,
                                                  int out_dtype, size_t count, nncase_hip_quant_param_t qp) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev, -EINVAL, "function_add_dequantize: null buffer");
    Op op;
    op.kind = Op::kDequantize;
    op.in0 = in_dev, op.out = out_dev, op.dt_in = in_dtype, op.dt_out = out_dtype, op.count = count, op.qp0 = qp;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qconv2d(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                               const nncase_hip_weights_t *weights, void *y_dev,
                                               const nncase_hip_conv2d_args_t *args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && weights && y_dev && args, -EINVAL, "function_add_qconv2d: null argument");
    Op op;
    op.kind = Op::kConv;
    op.in0 = x_dev, op.out = y_dev, op.weights = weights, op.conv = *args;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qblock(nncase_hip_function_t *fn, const uint8_t *x_dev, const nncase_hip_qblock_t *block,
                                              uint8_t *y_dev, const nncase_hip_qblock_args_t *args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && block && y_dev && args, -EINVAL, "function_add_qblock: null argument");
    Op op;
    op.kind = Op::kBlock;
    op.in0 = x_dev, op.out = y_dev, op.block = block, op.blk = *args;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qpointwise_pair(nncase_hip_function_t *fn, const uint8_t *x_dev, const nncase_hip_qpair_t *pair,
                                                       uint8_t *y1_dev, uint8_t *y2_dev, const nncase_hip_conv2d_args_t *first_args,
                                                       const nncase_hip_conv2d_args_t *second_args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && pair && y1_dev && y2_dev && first_args && second_args, -EINVAL,
                  "function_add_qpointwise_pair: null argument");
    Op op;
    op.kind = Op::kPair;
    op.in0 = x_dev, op.out = y1_dev, op.out2 = y2_dev, op.pair = pair, op.conv = *first_args, op.conv2 = *second_args;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qdepthwise_pointwise_pair(nncase_hip_function_t *fn, const uint8_t *x_dev,
                                                                 const nncase_hip_weights_t *depthwise,
                                                                 const nncase_hip_conv2d_args_t *depthwise_args, const nncase_hip_qpair_t *pair,
                                                                 uint8_t *y1_dev, uint8_t *y2_dev, const nncase_hip_conv2d_args_t *first_args,
                                                                 const nncase_hip_conv2d_args_t *second_args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && depthwise && depthwise_args && pair && y1_dev && y2_dev && first_args && second_args, -EINVAL,
                  "function_add_qdepthwise_pointwise_pair: null argument");
    Op op;
    op.kind = Op::kPair;
    op.in0 = x_dev, op.out = y1_dev, op.out2 = y2_dev, op.pair = pair, op.conv = *first_args, op.conv2 = *second_args;
    op.weights = depthwise, op.conv3 = *depthwise_args;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qglobal_avgpool_qconv2d(nncase_hip_function_t *fn, const uint8_t *x_dev, int32_t h, int32_t w,
                                                               nncase_hip_quant_param_t x_qp, const nncase_hip_weights_t *weights, void *y_dev,
                                                               const nncase_hip_conv2d_args_t *args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && weights && y_dev && args, -EINVAL, "function_add_qglobal_avgpool_qconv2d: null argument");
    Op op;
    op.kind = Op::kPoolConv;
    op.in0 = x_dev, op.out = y_dev, op.weights = weights, op.conv = *args, op.h = h, op.w = w, op.qp0 = x_qp;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qadd(nncase_hip_function_t *fn, const uint8_t *a_dev, nncase_hip_quant_param_t a_qp,
                                            const uint8_t *b_dev, nncase_hip_quant_param_t b_qp, uint8_t *out_dev,
                                            nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max, size_t count) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, a_dev && b_dev && out_dev, -EINVAL, "function_add_qadd: null buffer");
    Op op;
    op.kind = Op::kAdd;
    op.in0 = a_dev, op.in1 = b_dev, op.out = out_dev, op.qp0 = a_qp, op.qp1 = b_qp, op.qp2 = y_qp;
    op.lo = clamp_min, op.hi = clamp_max, op.count = count;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qglobal_avgpool(nncase_hip_function_t *fn, const uint8_t *x_dev, uint8_t *out_dev,
                                                       int32_t batch, int32_t h, int32_t w, int32_t channels,
                                                       nncase_hip_quant_param_t x_qp, nncase_hip_quant_param_t y_qp) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && out_dev, -EINVAL, "function_add_qglobal_avgpool: null buffer");
    Op op;
    op.kind = Op::kPool;
    op.in0 = x_dev, op.out = out_dev, op.batch = batch, op.h = h, op.w = w, op.channels = channels;
    op.qp0 = x_qp, op.qp1 = y_qp;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_lut_u8(nncase_hip_function_t *fn, const uint8_t *in_dev, uint8_t *out_dev,
                                              size_t count, const uint8_t *lut256_host) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev && lut256_host, -EINVAL, "function_add_lut_u8: null argument");
    Op op;
    op.kind = Op::kLut;
    op.in0 = in_dev, op.out = out_dev, op.count = count;
    memcpy(op.lut, lut256_host, 256);
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qconcat_channels(nncase_hip_function_t *fn, int32_t n_inputs,
                                                        const uint8_t *const *in_dev, const int32_t *channels,
                                                        const nncase_hip_quant_param_t *in_qps, uint8_t *out_dev,
                                                        nncase_hip_quant_param_t out_qp, int64_t pixels) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, n_inputs > 0 && n_inputs <= NNCASE_HIP_MAX_CONCAT && in_dev && channels && in_qps && out_dev,
                  -EINVAL, "function_add_qconcat_channels: bad argument (1..%d inputs)", NNCASE_HIP_MAX_CONCAT);
    Op op;
    op.kind = Op::kConcat;
    op.n_inputs = n_inputs, op.out = out_dev, op.qp0 = out_qp, op.pixels = pixels;
    for (int i = 0; i < n_inputs; i++) op.cat_in[i] = in_dev[i], op.cat_channels[i] = channels[i], op.cat_qp[i] = in_qps[i];
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_resize_nearest(nncase_hip_function_t *fn, const void *in_dev, void *out_dev,
                                                      int32_t elem_size, int32_t batch, int32_t in_h, int32_t in_w,
                                                      int32_t channels, int32_t out_h, int32_t out_w,
                                                      int32_t transformation_mode, int32_t nearest_mode) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev, -EINVAL, "function_add_resize_nearest: null buffer");
    Op op;
    op.kind = Op::kResize;
    op.in0 = in_dev, op.out = out_dev, op.elem_size = elem_size, op.batch = batch, op.h = in_h, op.w = in_w;
    op.channels = channels, op.out_h = out_h, op.out_w = out_w, op.tmode = transformation_mode, op.nmode = nearest_mode;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_layout(nncase_hip_function_t *fn, const void *in_dev, void *out_dev, int32_t elem_size,
                                              int32_t n, int32_t c, int32_t h, int32_t w, int32_t to_nchw) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev && in_dev != out_dev, -EINVAL, "function_add_layout: null or aliased buffers");
    NNHIP_REQUIRE(fn->ctx, (elem_size == 1 || elem_size == 2 || elem_size == 4) && n > 0 && c > 0 && h > 0 && w > 0 &&
                               (to_nchw == 0 || to_nchw == 1),
                  -EINVAL, "function_add_layout: bad arguments");
    Op op;
    op.kind = Op::kLayout;
    op.in0 = in_dev, op.out = out_dev, op.elem_size = elem_size, op.batch = n, op.channels = c, op.h = h, op.w = w;
    op.mode = to_nchw;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_qmaxpool2d(nncase_hip_function_t *fn, const uint8_t *x_dev, uint8_t *out_dev,
                                                  int32_t batch, int32_t in_h, int32_t in_w, int32_t channels,
                                                  int32_t kernel_h, int32_t kernel_w, int32_t stride_h, int32_t stride_w,
                                                  int32_t pad_h_before, int32_t pad_h_after, int32_t pad_w_before,
                                                  int32_t pad_w_after, nncase_hip_quant_param_t x_qp,
                                                  nncase_hip_quant_param_t y_qp) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && out_dev, -EINVAL, "function_add_qmaxpool2d: null buffer");
    Op op;
    op.kind = Op::kMaxPool;
    op.in0 = x_dev, op.out = out_dev, op.batch = batch, op.h = in_h, op.w = in_w, op.channels = channels;
    const int32_t v[8] = {kernel_h, kernel_w, stride_h, stride_w, pad_h_before, pad_h_after, pad_w_before, pad_w_after};
    memcpy(op.pool, v, sizeof(v));
    op.qp0 = x_qp, op.qp1 = y_qp;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_pack(nncase_hip_function_t *fn, const void *in_dev, void *out_dev, int32_t elem_size,
                                            int32_t rank, const int32_t *shape, int32_t n_axes, const int32_t *axes,
                                            const int32_t *lanes) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev && shape && rank > 0 && rank <= 8 && n_axes >= 0 && n_axes <= 8 &&
                               (n_axes == 0 || (axes && lanes)),
                  -EINVAL, "function_add_pack: bad argument");
    Op op;
    op.kind = Op::kPack;
    op.in0 = in_dev, op.out = out_dev, op.elem_size = elem_size, op.rank = rank, op.n_axes = n_axes;
    for (int i = 0; i < rank; i++) op.shape[i] = shape[i];
    for (int i = 0; i < n_axes; i++) op.axes[i] = axes[i], op.lanes[i] = lanes[i];
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_quantize_pack(nncase_hip_function_t *fn, const float *in_dev, uint8_t *out_dev, int32_t rank,
                                                     const int32_t *shape, int32_t n_axes, const int32_t *axes, const int32_t *lanes,
                                                     nncase_hip_quant_param_t qp) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, in_dev && out_dev && shape && rank > 0 && rank <= 8 && n_axes > 0 && n_axes <= 8 && axes && lanes, -EINVAL,
                  "function_add_quantize_pack: bad argument");
    Op op;
    op.kind = Op::kQuantPack;
    op.in0 = in_dev, op.out = out_dev, op.rank = rank, op.n_axes = n_axes, op.qp0 = qp;
    for (int i = 0; i < rank; i++) op.shape[i] = shape[i];
    for (int i = 0; i < n_axes; i++) op.axes[i] = axes[i], op.lanes[i] = lanes[i];
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_w8a16_gemm(nncase_hip_function_t *fn, const void *a_dev, const nncase_hip_w8a16_t *weights,
                                                  void *out_dev, int32_t m, int32_t mode, const void *residual_dev,
                                                  int32_t out_dtype) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, a_dev && weights && out_dev, -EINVAL, "function_add_w8a16_gemm: null argument");
    Op op;
    op.kind = Op::kGemm;
    op.in0 = a_dev, op.w8 = weights, op.out = out_dev, op.batch = m, op.mode = mode, op.in1 = residual_dev, op.dt_out = out_dtype;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_rmsnorm_w8a16_gemm(nncase_hip_function_t *fn, const void *x_dev, const void *ln_weight_dev,
                                                          float eps, const nncase_hip_w8a16_t *weights, void *out_dev, int32_t m,
                                                          int32_t mode, const void *residual_dev, int32_t out_dtype) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && ln_weight_dev && weights && out_dev, -EINVAL, "function_add_rmsnorm_w8a16_gemm: null argument");
    Op op;
    op.kind = Op::kGemm;
    op.in0 = x_dev, op.in2 = ln_weight_dev, op.eps = eps, op.w8 = weights, op.out = out_dev, op.batch = m, op.mode = mode;
    op.in1 = residual_dev, op.dt_out = out_dtype;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_rmsnorm_f16(nncase_hip_function_t *fn, const void *x_dev, const void *weight_dev,
                                                   void *out_dev, int32_t rows, int32_t hidden, float eps) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && weight_dev && out_dev, -EINVAL, "function_add_rmsnorm_f16: null argument");
    Op op;
    op.kind = Op::kRmsNorm;
    op.in0 = x_dev, op.in1 = weight_dev, op.out = out_dev, op.batch = rows, op.channels = hidden, op.eps = eps;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_rope_kv_append(nncase_hip_function_t *fn, const void *qkv_dev, void *q_out_dev,
                                                      void *k_cache_dev, void *v_cache_dev, const int32_t *block_table_dev,
                                                      const int32_t *ctx_lens_dev, const nncase_hip_paged_attn_args_t *geometry,
                                                      float rope_theta) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, qkv_dev && q_out_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && geometry, -EINVAL,
                  "function_add_rope_kv_append: null argument");
    Op op;
    op.kind = Op::kRope;
    op.in0 = qkv_dev, op.out = q_out_dev, op.out2 = k_cache_dev, op.out3 = v_cache_dev, op.in2 = block_table_dev, op.in3 = ctx_lens_dev;
    op.attn = *geometry, op.eps = rope_theta;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_w8a16_gemm_rope_kv_append(nncase_hip_function_t *fn, const void *x_dev, const void *ln_weight_dev,
                                                                 float eps, const nncase_hip_w8a16_t *weights, void *qkv_dev,
                                                                 void *q_out_dev, void *k_cache_dev, void *v_cache_dev,
                                                                 const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                                                 const nncase_hip_paged_attn_args_t *geometry, float rope_theta) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && weights && qkv_dev && q_out_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && geometry,
                  -EINVAL, "function_add_w8a16_gemm_rope_kv_append: null argument");
    Op op;
    op.kind = Op::kGemmRope;
    op.in0 = x_dev, op.in1 = ln_weight_dev, op.eps = eps, op.w8 = weights, op.out = qkv_dev, op.in4 = q_out_dev;
    op.out2 = k_cache_dev, op.out3 = v_cache_dev, op.in2 = block_table_dev, op.in3 = ctx_lens_dev;
    op.attn = *geometry, op.theta = rope_theta;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_paged_attention_decode(nncase_hip_function_t *fn, const void *q_dev, const void *k_cache_dev,
                                                              const void *v_cache_dev, const int32_t *block_table_dev,
                                                              const int32_t *ctx_lens_dev, void *out_dev,
                                                              const nncase_hip_paged_attn_args_t *args) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, q_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && out_dev && args, -EINVAL,
                  "function_add_paged_attention_decode: null argument");
    // the workspace the kernel's splits go through is sized now: capture must not allocate, and a graph
    // keeps the addresses it was captured with
    const int lane = fn->cur_lane;
    if (lane <= 0) { // (lane 0, and behind the join, where lane 0 has finished: the context's scratch)
        const int rc = attn_reserve(fn->ctx, args);
        if (rc) return rc;
    } else {
        size_t pb = 0, cb = 0;
        const int rc = attn_scratch_sizes(fn->ctx, args, &pb, &cb);
        if (rc) return rc;
        if (pb > fn->lane_partial_bytes[lane] || cb > fn->lane_counter_bytes[lane]) {
            NNHIP_REQUIRE(fn->ctx, !fn->exec, -EBUSY, "function_add_paged_attention_decode: the lane's scratch would grow under a captured graph");
            NNHIP_HIP(fn->ctx, hipStreamSynchronize(fn->ctx->stream)); // earlier eager invocations may still use the old areas
            if (pb > fn->lane_partial_bytes[lane]) {
                if (fn->lane_partials[lane]) NNHIP_HIP(fn->ctx, hipFree(fn->lane_partials[lane]));
                fn->lane_partials[lane] = nullptr, fn->lane_partial_bytes[lane] = 0;
                NNHIP_HIP(fn->ctx, hipMalloc(&fn->lane_partials[lane], pb));
                fn->lane_partial_bytes[lane] = pb;
            }
            if (cb > fn->lane_counter_bytes[lane]) {
                if (fn->lane_counters[lane]) NNHIP_HIP(fn->ctx, hipFree(fn->lane_counters[lane]));
                fn->lane_counters[lane] = nullptr, fn->lane_counter_bytes[lane] = 0;
                const size_t cap = (cb + 4095) / 4096 * 4096;
                NNHIP_HIP(fn->ctx, hipMalloc(&fn->lane_counters[lane], cap));
                fn->lane_counter_bytes[lane] = cap;
                NNHIP_HIP(fn->ctx, hipMemset(fn->lane_counters[lane], 0, cap)); // (not under capture: recording comes first)
            }
        }
    }
    Op op;
    op.kind = Op::kAttn;
    op.in0 = q_dev, op.in1 = k_cache_dev, op.in2 = v_cache_dev, op.in3 = block_table_dev, op.in4 = ctx_lens_dev, op.out = out_dev;
    op.attn = *args;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_argmax_f32(nncase_hip_function_t *fn, const float *x_dev, int32_t *out_dev, int32_t rows,
                                                  int32_t cols) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev && out_dev, -EINVAL, "function_add_argmax_f32: null argument");
    Op op;
    op.kind = Op::kArgmax;
    op.in0 = x_dev, op.out = out_dev, op.batch = rows, op.channels = cols;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_embedding_f16(nncase_hip_function_t *fn, const void *table_dev, const int32_t *ids_dev,
                                                     void *out_dev, int32_t rows, int32_t hidden, int32_t vocab) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, table_dev && ids_dev && out_dev, -EINVAL, "function_add_embedding_f16: null argument");
    Op op;
    op.kind = Op::kEmbed;
    op.in0 = table_dev, op.in1 = ids_dev, op.out = out_dev, op.batch = rows, op.channels = hidden, op.w = vocab;
    return push(fn, op);
}

extern "C" int nncase_hip_function_add_add_i32(nncase_hip_function_t *fn, int32_t *x_dev, int32_t count, int32_t delta) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, x_dev, -EINVAL, "function_add_add_i32: null argument");
    Op op;
    op.kind = Op::kAddI32;
    op.out = x_dev, op.batch = count, op.delta = delta;
    return push(fn, op);
}

extern "C" int nncase_hip_function_size(nncase_hip_function_t *fn, int32_t *count) {
    if (!fn || !count) return -EINVAL;
    *count = (int32_t)fn->ops.size();
    return 0;
}

extern "C" int nncase_hip_function_invoke_one(nncase_hip_function_t *fn, int32_t index) {
    if (!fn) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, index >= 0 && (size_t)index < fn->ops.size(), -EINVAL, "function_invoke_one: index %d of %zu",
                  index, fn->ops.size());
    return run_op(fn, fn->ops[index]);
}

extern "C" int nncase_hip_function_invoke(nncase_hip_function_t *fn) {
    if (!fn) return -EINVAL;
    if (fn->exec) {
        NNHIP_HIP(fn->ctx, hipGraphLaunch(fn->exec, fn->ctx->stream));
        return 0;
    }
    for (const Op &op : fn->ops) {
        const int rc = run_op(fn, op);
        if (rc) return rc;
    }
    return 0;
}

extern "C" int nncase_hip_function_capture(nncase_hip_function_t *fn) {
    if (!fn) return -EINVAL;
    nncase_hip_ctx *ctx = fn->ctx;
    drop_graph(fn);
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    // (paged attention on lane 0 goes through the context's scratch area, whose addresses the graph will hold;
    // other lanes bring areas of their own)
    int attn_lane = -1;
    for (const Op &op : fn->ops)
        if (op.kind == Op::kAttn && op.lane <= 0) attn_lane = 0;
    // Operators of different lanes are recorded on streams of their own, forked from and joined back into
    // the context's stream, so the graph holds one independent chain per lane and the device overlaps them.
    hipStream_t main_stream = ctx->stream;
    hipStream_t side[NNCASE_HIP_MAX_LANES] = {nullptr};
    hipEvent_t fork = nullptr, join[NNCASE_HIP_MAX_LANES] = {nullptr};
    int rc = 0;
    hipError_t se = hipSuccess;
    for (int l = 1; l < fn->nlanes && se == hipSuccess; l++) {
        se = hipStreamCreateWithFlags(&side[l], hipStreamNonBlocking);
        if (se == hipSuccess) se = hipEventCreateWithFlags(&join[l], hipEventDisableTiming);
    }
    if (se == hipSuccess && fn->nlanes > 1) se = hipEventCreateWithFlags(&fork, hipEventDisableTiming);
    auto release = [&]() {
        for (int l = 1; l < NNCASE_HIP_MAX_LANES; l++) {
            if (join[l]) (void)hipEventDestroy(join[l]);
            if (side[l]) (void)hipStreamDestroy(side[l]);
        }
        if (fork) (void)hipEventDestroy(fork);
    };
    if (se != hipSuccess) {
        release();
        return hip_fail(ctx, se, "function_capture: lane streams");
    }
    se = hipStreamBeginCapture(main_stream, hipStreamCaptureModeThreadLocal);
    if (se != hipSuccess) {
        release();
        return hip_fail(ctx, se, "hipStreamBeginCapture");
    }
    if (fn->nlanes > 1) {
        se = hipEventRecord(fork, main_stream);
        for (int l = 1; l < fn->nlanes && se == hipSuccess; l++) se = hipStreamWaitEvent(side[l], fork, 0);
    }
    if (se == hipSuccess) {
        for (const Op &op : fn->ops) {
            if (op.lane == NNCASE_HIP_LANE_JOINED) continue;
            ctx->stream = op.lane == 0 ? main_stream : side[op.lane];
            rc = run_op(fn, op);
            if (rc) break;
        }
        ctx->stream = main_stream;
        for (int l = 1; l < fn->nlanes && se == hipSuccess; l++) {
            se = hipEventRecord(join[l], side[l]);
            if (se == hipSuccess) se = hipStreamWaitEvent(main_stream, join[l], 0);
        }
        // what was recorded behind the join: on the context's stream, after every lane
        for (const Op &op : fn->ops) {
            if (rc || se != hipSuccess) break;
            if (op.lane == NNCASE_HIP_LANE_JOINED) rc = run_op(fn, op);
        }
    }
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(main_stream, &graph);
    release();
    if (se != hipSuccess && !rc) rc = hip_fail(ctx, se, "function_capture: fork / join");
    if (rc) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    NNHIP_HIP(ctx, e);
    fn->graph = graph;
    const hipError_t ie = hipGraphInstantiate(&fn->exec, fn->graph, nullptr, nullptr, 0);
    if (ie != hipSuccess) {
        drop_graph(fn);
        return hip_fail(ctx, ie, "hipGraphInstantiate");
    }
    if (attn_lane >= 0) {
        fn->pins_attn = true;
        ctx->attn_pins++;
    }
    return 0;
}

extern "C" int nncase_hip_function_op_kernel(nncase_hip_function_t *fn, int32_t index, char *name, size_t capacity) {
    if (!fn || !name || capacity == 0) return -EINVAL;
    NNHIP_REQUIRE(fn->ctx, index >= 0 && (size_t)index < fn->ops.size(), -EINVAL, "function_op_kernel: index %d of %zu", index,
                  fn->ops.size());
    const Op &op = fn->ops[index];
    switch (op.kind) {
    case Op::kQuantize: snprintf(name, capacity, "quantize"); break;
    case Op::kDequantize: snprintf(name, capacity, "dequantize"); break;
    case Op::kConv: describe_conv_kernel(fn->ctx, op.weights, &op.conv, name, capacity); break;
    case Op::kBlock: nncase_hip_qblock_describe(op.block, &op.blk, name, capacity); break;
    case Op::kPoolConv: snprintf(name, capacity, "qglobal_avgpool+qpointwise_rows%s", op.conv.dequantize_output ? "+dequantize" : ""); break;
    case Op::kPair: snprintf(name, capacity, op.weights ? "dw3x3+qpointwise_pair_kernel" : "qpointwise_pair_kernel"); break;
    case Op::kAdd: snprintf(name, capacity, "qadd"); break;
    case Op::kPool: snprintf(name, capacity, "qglobal_avgpool"); break;
    case Op::kLut: snprintf(name, capacity, "lut_u8"); break;
    case Op::kConcat: snprintf(name, capacity, "qconcat<%d>", op.n_inputs); break;
    case Op::kResize: snprintf(name, capacity, "resize_nearest"); break;
    case Op::kLayout: snprintf(name, capacity, op.mode ? "nhwc_to_nchw" : "nchw_to_nhwc"); break;
    case Op::kMaxPool: snprintf(name, capacity, "qmaxpool<%dx%d>", op.pool[0], op.pool[1]); break;
    case Op::kPack: snprintf(name, capacity, "pack"); break;
    case Op::kQuantPack: snprintf(name, capacity, "quantize+pack"); break;
    case Op::kGemm:
        snprintf(name, capacity, "%sw8a16_gemm%s", op.in2 ? "rmsnorm+" : "",
                 op.mode == NNCASE_HIP_GEMM_SWIGLU ? "+swiglu" : (op.in1 ? "+residual" : ""));
        break;
    case Op::kRmsNorm: snprintf(name, capacity, "rmsnorm_f16"); break;
    case Op::kRope: snprintf(name, capacity, "rope_kv_append"); break;
    case Op::kGemmRope: snprintf(name, capacity, "%sw8a16_gemm+rope_kv_append", op.in1 ? "rmsnorm+" : ""); break;
    case Op::kAttn: snprintf(name, capacity, "paged_attention_decode"); break;
    case Op::kArgmax: snprintf(name, capacity, "argmax_f32"); break;
    case Op::kEmbed: snprintf(name, capacity, "embedding_f16"); break;
    case Op::kAddI32: snprintf(name, capacity, "add_i32"); break;
    }
    return 0;
}

extern "C" int nncase_hip_function_profile(nncase_hip_function_t *fn, int32_t iterations, float *avg_ms) {
    if (!fn || !avg_ms) return -EINVAL;
    nncase_hip_ctx *ctx = fn->ctx;
    NNHIP_REQUIRE(ctx, iterations > 0, -EINVAL, "function_profile: iterations must be positive");
    hipEvent_t e0, e1;
    NNHIP_HIP(ctx, hipEventCreate(&e0));
    NNHIP_HIP(ctx, hipEventCreate(&e1));
    int rc = 0;
    for (size_t i = 0; i < fn->ops.size() && rc == 0; i++) {
        rc = run_op(fn, fn->ops[i]); // warm
        if (rc) break;
        hipError_t e = hipEventRecord(e0, ctx->stream);
        for (int it = 0; it < iterations && rc == 0; it++) rc = run_op(fn, fn->ops[i]);
        if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess && rc == 0) rc = hip_fail(ctx, e, "function_profile");
        avg_ms[i] = ms / (float)iterations;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}
