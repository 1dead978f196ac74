// Native loader for kmodel v7 files whose entry function lives in a module of kind "hip".
//
// Container (all little-endian; src/Native/include/nncase/runtime/model.h:38-74, reader order of
// src/Native/src/runtime/interpreter.cpp:40-91 and runtime_module.cpp:124-180):
//   model_header, then per module: module_header, functions (function_header, parameter and
//   return type signatures, function sections), module sections; every `size` field covers its
//   header and body, so modules / functions / sections are skipped by size.
// The hip module keeps its operator list in the module section ".text" (the function header's
// entrypoint / text_size select the function's slice, as for the stackvm module) and its
// constants in ".rdata".  Loading uploads and pre-packs the constants, allocates one device
// buffer per tensor and records the operators into a resident function, which is what the
// module's runtime_function::invoke_core would run (src/Native/include/nncase/runtime/
// runtime_function.h:55-63).
#include "qconv.hpp"

#include <memory>
#include <new>
#include <string>
#include <vector>

namespace {

#pragma pack(push, 1)
struct model_header {
    uint32_t identifier, version, flags, alignment, modules, entry_module, entry_function, reserved0;
};
struct module_header {
    char kind[16];
    uint32_t version, sections, functions, reserved0;
    uint64_t size;
};
struct function_header {
    uint32_t parameters, sections;
    uint64_t entrypoint, text_size, size;
};
struct section_header {
    char name[16];
    uint32_t flags, reserved0;
    uint64_t size, body_start, body_size, memory_size;
};
struct hipf_header {
    char magic[4];
    uint32_t version, n_tensors, n_ops, input_tensor, output_tensor, n_outputs, reserved;
};
struct hipf_tensor {
    uint32_t dtype, rank, dims[4];
    int32_t zero_point;
    float scale;
};
struct hipf_op {
    uint32_t opcode, n_inputs;
    int32_t inputs[8];
    int32_t output;
    uint32_t reserved;
    uint64_t rdata0, rdata1;
    int32_t p[16];
    float f[4];
};
#pragma pack(pop)
static_assert(sizeof(model_header) == 32 && sizeof(module_header) == 40 && sizeof(function_header) == 32 &&
                  sizeof(section_header) == 56,
              "kmodel v7 header sizes");
static_assert(sizeof(hipf_header) == 32 && sizeof(hipf_tensor) == 32 && sizeof(hipf_op) == 144, "hip text record sizes");

constexpr uint32_t kModelIdentifier = 0x4B4D444C; // 'KMDL'
constexpr uint32_t kModelVersion = 7;
constexpr uint64_t kNoRdata = ~uint64_t(0);
enum { kOpQuantize, kOpDequantize, kOpConv2d, kOpAdd, kOpGlobalAvgPool, kOpLut, kOpConcat, kOpResizeNearest, kOpMaxPool,
       kOpPadChannels, kOpReshape, kOpLayout };

struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
};

size_t dtype_size(uint32_t dt) {
    switch (dt) {
    case NNCASE_HIP_DT_U8:
    case NNCASE_HIP_DT_I8: return 1;
    case NNCASE_HIP_DT_I16:
    case NNCASE_HIP_DT_F16: return 2;
    case NNCASE_HIP_DT_I32:
    case NNCASE_HIP_DT_F32: return 4;
    default: return 0;
    }
}

} // namespace

struct nncase_hip_kmodel {
    nncase_hip_ctx *ctx = nullptr;
    std::vector<hipf_tensor> tensors;
    std::vector<void *> buffers;      // one device buffer per tensor (aliases share an entry's value)
    std::vector<char> owns;           // whether buffers[i] is freed with the model
    std::vector<nncase_hip_weights_t *> weights;
    std::vector<nncase_hip_qblock_t *> blocks;
    std::vector<nncase_hip_qpair_t *> pairs; // (point at entries of `weights`: destroyed first)
    nncase_hip_function_t *fn = nullptr;
    uint32_t input_tensor = 0, output_tensor = 0, n_outputs = 1; // outputs are consecutive tensors
};

using namespace nnhip;

extern "C" int nncase_hip_kmodel_destroy(nncase_hip_kmodel_t *m) {
    if (!m) return -EINVAL;
    if (m->fn) (void)nncase_hip_function_destroy(m->fn); // synchronises the stream first
    for (auto *pr : m->pairs)
        if (pr) (void)nncase_hip_qpointwise_pair_destroy(m->ctx, pr);
    for (auto *w : m->weights)
        if (w) (void)nncase_hip_weights_destroy(m->ctx, w);
    for (auto *b : m->blocks)
        if (b) (void)nncase_hip_qblock_destroy(m->ctx, b);
    for (size_t i = 0; i < m->buffers.size(); i++)
        if (m->owns[i] && m->buffers[i]) (void)hipFree(m->buffers[i]);
    delete m;
    return 0;
}

// Finds section `name` among `count` section records starting at `pos`, as runtime::find_section does
// (src/Native/src/runtime/section.cpp:58-91): the body starts body_start bytes behind the section
// header (the writer stores the alignment padding there, src/Nncase.CodeGen/CodeGen/LinkedModel.cs:160),
// or, for a section flagged SECTION_MERGED_INTO_RDATA (model.h:76), body_start bytes into the body of
// the list's ".rdata" section.
static bool find_section(const uint8_t *file, size_t size, size_t first, uint32_t count, const char *name, Span *out, int depth = 0) {
    size_t pos = first;
    for (uint32_t i = 0; i < count; i++) {
        if (pos + sizeof(section_header) > size) return false;
        section_header h;
        memcpy(&h, file + pos, sizeof(h));
        if (h.size < sizeof(h) || h.size > size - pos) return false;
        if (strncmp(h.name, name, 16) == 0) {
            if (h.flags & 1u) { // merged into .rdata
                Span rdata;
                if (depth > 0 || !find_section(file, size, first, count, ".rdata", &rdata, depth + 1)) return false;
                if (h.body_start > rdata.n || h.body_size > rdata.n - h.body_start) return false;
                out->p = rdata.p + h.body_start;
                out->n = (size_t)h.body_size;
                return true;
            }
            const size_t body0 = pos + sizeof(section_header);
            if (h.body_start > size - body0 || h.body_size > size - body0 - h.body_start) return false;
            out->p = file + body0 + (size_t)h.body_start;
            out->n = (size_t)h.body_size;
            return true;
        }
        pos += (size_t)h.size;
    }
    return false;
}

static int build_function(nncase_hip_ctx_t *ctx, Span text_span, Span rdata, nncase_hip_kmodel_t **out);

extern "C" int nncase_hip_kmodel_load(nncase_hip_ctx_t *ctx, const void *data, size_t size, nncase_hip_kmodel_t **out) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, data && out, -EINVAL, "kmodel_load: null argument");
    *out = nullptr;
    const uint8_t *file = static_cast<const uint8_t *>(data);
    NNHIP_REQUIRE(ctx, size >= sizeof(model_header), -EINVAL, "kmodel_load: file shorter than a model header");
    model_header mh;
    memcpy(&mh, file, sizeof(mh));
    // the two checks of interpreter::initialize_model (src/Native/src/runtime/interpreter.cpp:95-102)
    NNHIP_REQUIRE(ctx, mh.identifier == kModelIdentifier, -NNCASE_HIP_ERR_INVALID_MODEL_IDENTIFIER,
                  "kmodel_load: invalid model identifier 0x%08x", mh.identifier);
    NNHIP_REQUIRE(ctx, mh.version == kModelVersion, -NNCASE_HIP_ERR_INVALID_MODEL_VERSION,
                  "kmodel_load: model version %u (this runtime reads version %u)", mh.version, kModelVersion);
    NNHIP_REQUIRE(ctx, mh.entry_module != 0xFFFFFFFFu && mh.entry_module < mh.modules, -EINVAL,
                  "kmodel_load: model has no entry function");

    // ---- locate the hip function ------------------------------------------------------------------
    // Modules are skipped by their size field (interpreter.cpp:55-70), functions likewise
    // (skip_functions, runtime_module.cpp:112-117); the module sections follow the functions.
    struct Located {
        module_header modh{};
        function_header fh{};
        size_t sections_pos = 0;
    };
    auto locate = [&](uint32_t module_id, uint32_t function_id, Located *loc) -> int {
        NNHIP_REQUIRE(ctx, module_id < mh.modules, -NNCASE_HIP_ERR_RUNTIME_NOT_FOUND, "kmodel_load: module %u of %u", module_id,
                      mh.modules);
        size_t pos = sizeof(model_header);
        for (uint32_t i = 0;; i++) {
            NNHIP_REQUIRE(ctx, pos + sizeof(module_header) <= size, -EINVAL, "kmodel_load: truncated module header");
            memcpy(&loc->modh, file + pos, sizeof(module_header));
            NNHIP_REQUIRE(ctx, loc->modh.size >= sizeof(module_header) && loc->modh.size <= size - pos, -EINVAL,
                          "kmodel_load: bad module size");
            if (i == module_id) break;
            pos += (size_t)loc->modh.size;
        }
        NNHIP_REQUIRE(ctx, function_id < loc->modh.functions, -EINVAL, "kmodel_load: function %u of %u in module %u",
                      function_id, loc->modh.functions, module_id);
        const size_t module_end = pos + (size_t)loc->modh.size;
        size_t fpos = pos + sizeof(module_header);
        for (uint32_t i = 0; i < loc->modh.functions; i++) {
            NNHIP_REQUIRE(ctx, fpos + sizeof(function_header) <= module_end, -EINVAL, "kmodel_load: truncated function header");
            function_header h;
            memcpy(&h, file + fpos, sizeof(h));
            NNHIP_REQUIRE(ctx, h.size >= sizeof(h) && h.size <= module_end - fpos, -EINVAL, "kmodel_load: bad function size");
            if (i == function_id) loc->fh = h;
            fpos += (size_t)h.size;
        }
        loc->sections_pos = fpos;
        return 0;
    };
    auto function_text = [&](const Located &loc, Span *text, Span *rdata) -> int {
        Span text_all;
        NNHIP_REQUIRE(ctx, find_section(file, size, loc.sections_pos, loc.modh.sections, ".text", &text_all), -EINVAL,
                      "kmodel_load: module \"%.16s\" has no .text section", loc.modh.kind);
        if (!find_section(file, size, loc.sections_pos, loc.modh.sections, ".rdata", rdata)) *rdata = Span{};
        NNHIP_REQUIRE(ctx, loc.fh.entrypoint <= text_all.n && loc.fh.text_size <= text_all.n - loc.fh.entrypoint, -EINVAL,
                      "kmodel_load: function text outside the .text section");
        text->p = text_all.p + loc.fh.entrypoint;
        text->n = (size_t)loc.fh.text_size;
        return 0;
    };
    Located loc;
    int lrc = locate(mh.entry_module, mh.entry_function, &loc);
    if (lrc) return lrc;
    Span text_span, rdata;
    if (strncmp(loc.modh.kind, "stackvm", 16) == 0) {
        // A compiled kmodel's entry is a stackvm function; the only one this loader runs is the call
        // stub the compiler emits around a function of another module
        // (modules/Nncase.Modules.StackVM/CodeGen/StackVM/CodegenVisitor.cs:281-315,470-476):
        //   LDARG n-1 .. LDARG 0 ; LDC_I4 function id ; LDC_I4 module id ; EXTCALL args, is_prim_func ; RET
        // with the encodings of src/Native/include/nncase/runtime/stackvm/op_reader.h:59-64,83-90,116-122,386-392
        // (opcode byte, operands unaligned little-endian) and EXTCALL's pop order of
        // src/Native/src/runtime/stackvm/ops/control.cpp:25-47.  Any other text needs the stackvm
        // interpreter, which is not this library.
        Span sv, sv_rdata;
        lrc = function_text(loc, &sv, &sv_rdata);
        if (lrc) return lrc;
        size_t pc = 0;
        auto rd = [&](void *dst, size_t n) {
            if (pc + n > sv.n) return false;
            memcpy(dst, sv.p + pc, n);
            pc += n;
            return true;
        };
        uint32_t n_ldarg = 0;
        bool ok = true;
        for (;;) { // arguments are pushed last first, so that EXTCALL pops them in declaration order
            uint8_t opc = 0;
            if (pc >= sv.n) { ok = false; break; }
            opc = sv.p[pc];
            uint16_t index = 0;
            if (opc == 39) { // LDARG u16
                pc++;
                if (!rd(&index, 2)) { ok = false; break; }
            } else if (opc >= 40 && opc <= 45) { // LDARG_0 .. LDARG_5
                pc++;
                index = (uint16_t)(opc - 40);
            } else
                break;
            n_ldarg++;
            if (index != loc.fh.parameters - n_ldarg) { ok = false; break; }
        }
        uint8_t opc = 0;
        int32_t func_id = -1, module_id = -1;
        uint16_t call_args = 0;
        uint8_t is_prim = 0;
        ok = ok && n_ldarg == loc.fh.parameters && rd(&opc, 1) && opc == 2 && rd(&func_id, 4) && rd(&opc, 1) && opc == 2 &&
             rd(&module_id, 4) && rd(&opc, 1) && opc == 96 && rd(&call_args, 2) && rd(&is_prim, 1) && rd(&opc, 1) && opc == 93 &&
             pc == sv.n && call_args == n_ldarg && is_prim <= 1 && func_id >= 0 && module_id >= 0;
        NNHIP_REQUIRE(ctx, ok, -NNCASE_HIP_ERR_RUNTIME_NOT_FOUND,
                      "kmodel_load: the stackvm entry function is not a plain call into another module (this library runs "
                      "hip functions, not stackvm code)");
        NNHIP_REQUIRE(ctx, (uint32_t)module_id != mh.entry_module, -NNCASE_HIP_ERR_RUNTIME_NOT_FOUND,
                      "kmodel_load: the stackvm entry function calls its own module");
        const uint32_t caller_args = n_ldarg;
        lrc = locate((uint32_t)module_id, (uint32_t)func_id, &loc);
        if (lrc) return lrc;
        // a prim function receives its outputs as trailing parameters (control.cpp:49-68)
        NNHIP_REQUIRE(ctx, is_prim ? loc.fh.parameters > caller_args : loc.fh.parameters == caller_args, -EINVAL,
                      "kmodel_load: EXTCALL passes %u arguments to a function of %u parameters", caller_args, loc.fh.parameters);
    }
    NNHIP_REQUIRE(ctx, strncmp(loc.modh.kind, "hip", 16) == 0, -NNCASE_HIP_ERR_RUNTIME_NOT_FOUND,
                  "kmodel_load: module kind \"%.16s\" is not \"hip\"", loc.modh.kind);
    lrc = function_text(loc, &text_span, &rdata);
    if (lrc) return lrc;
    return build_function(ctx, text_span, rdata, out);
}

// One function of a hip module from the two byte ranges the reference's runtime hands a runtime_function:
// its slice of the module's .text section (function_header::entrypoint, text_size) and the module's .rdata
// section (the stackvm module reads the same pair, src/Native/src/runtime/stackvm/runtime_module.cpp:27-30,
// runtime_function.cpp:31-36).
extern "C" int nncase_hip_kmodel_load_function(nncase_hip_ctx_t *ctx, const void *text, size_t text_size, const void *rdata,
                                               size_t rdata_size, nncase_hip_kmodel_t **out) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, text && out && (rdata || rdata_size == 0), -EINVAL, "kmodel_load_function: null argument");
    *out = nullptr;
    return build_function(ctx, Span{static_cast<const uint8_t *>(text), text_size},
                          Span{static_cast<const uint8_t *>(rdata), rdata_size}, out);
}

static int build_function(nncase_hip_ctx_t *ctx, Span text_span, Span rdata, nncase_hip_kmodel_t **out) {
    const uint8_t *text = text_span.p;
    const size_t text_size = text_span.n;

    // ---- function text --------------------------------------------------------------------------
    NNHIP_REQUIRE(ctx, text_size >= sizeof(hipf_header), -EINVAL, "kmodel_load: function text too short");
    hipf_header th;
    memcpy(&th, text, sizeof(th));
    NNHIP_REQUIRE(ctx, memcmp(th.magic, "HIPF", 4) == 0 && th.version == 1, -EINVAL, "kmodel_load: not a hip function text");
    NNHIP_REQUIRE(ctx, th.n_tensors <= (1u << 20) && th.n_ops <= (1u << 20), -EINVAL, "kmodel_load: implausible counts");
    const size_t need = sizeof(hipf_header) + (size_t)th.n_tensors * sizeof(hipf_tensor) + (size_t)th.n_ops * sizeof(hipf_op);
    NNHIP_REQUIRE(ctx, need <= text_size, -EINVAL, "kmodel_load: function text truncated");
    const uint32_t n_outputs = th.n_outputs ? th.n_outputs : 1;
    NNHIP_REQUIRE(ctx, th.input_tensor < th.n_tensors && th.output_tensor < th.n_tensors &&
                           n_outputs <= th.n_tensors - th.output_tensor,
                  -EINVAL, "kmodel_load: input / output tensor index out of range");

    std::unique_ptr<nncase_hip_kmodel, int (*)(nncase_hip_kmodel *)> m(new (std::nothrow) nncase_hip_kmodel(),
                                                                      nncase_hip_kmodel_destroy);
    NNHIP_REQUIRE(ctx, m, -ENOMEM, "kmodel_load: out of host memory");
    m->ctx = ctx;
    m->input_tensor = th.input_tensor, m->output_tensor = th.output_tensor, m->n_outputs = n_outputs;
    m->tensors.resize(th.n_tensors);
    memcpy(m->tensors.data(), text + sizeof(hipf_header), (size_t)th.n_tensors * sizeof(hipf_tensor));
    std::vector<hipf_op> ops(th.n_ops);
    memcpy(ops.data(), text + sizeof(hipf_header) + (size_t)th.n_tensors * sizeof(hipf_tensor), (size_t)th.n_ops * sizeof(hipf_op));

    auto elems = [&](uint32_t t) {
        const hipf_tensor &x = m->tensors[t];
        return (size_t)x.dims[0] * x.dims[1] * x.dims[2] * x.dims[3];
    };
    auto tqp = [&](uint32_t t) { return nncase_hip_quant_param_t{m->tensors[t].zero_point, m->tensors[t].scale}; };
    for (uint32_t t = 0; t < th.n_tensors; t++) {
        const hipf_tensor &x = m->tensors[t];
        NNHIP_REQUIRE(ctx, x.rank == 4 && dtype_size(x.dtype) != 0, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                      "kmodel_load: tensor %u has rank %u / dtype 0x%x", t, x.rank, x.dtype);
        // four 32-bit extents can wrap a 64-bit product: bound every extent and every partial product
        // (2^24 * 2^40 < 2^64, so the running product cannot wrap before it is checked)
        bool sane = true;
        uint64_t prod = 1;
        for (int d = 0; d < 4 && sane; d++) {
            sane = x.dims[d] != 0 && x.dims[d] <= (1u << 24);
            prod *= x.dims[d];
            sane = sane && prod < (uint64_t(1) << 40);
        }
        NNHIP_REQUIRE(ctx, sane, -EINVAL, "kmodel_load: tensor %u has an empty or implausible shape", t);
    }

    // ---- which adds fold into the dense conv right before them -------------------------------
    std::vector<int> consumers(th.n_tensors, 0), producer(th.n_tensors, -1);
    for (uint32_t k = 0; k < th.n_ops; k++) {
        const hipf_op &o = ops[k];
        NNHIP_REQUIRE(ctx, o.n_inputs >= 1 && o.n_inputs <= 8 && o.output >= 0 && (uint32_t)o.output < th.n_tensors, -EINVAL,
                      "kmodel_load: operator %u has bad operand counts", k);
        for (uint32_t i = 0; i < o.n_inputs; i++) {
            NNHIP_REQUIRE(ctx, o.inputs[i] >= 0 && (uint32_t)o.inputs[i] < th.n_tensors, -EINVAL,
                          "kmodel_load: operator %u reads tensor %d", k, o.inputs[i]);
            NNHIP_REQUIRE(ctx, (uint32_t)o.inputs[i] == th.input_tensor || producer[o.inputs[i]] >= 0, -EINVAL,
                          "kmodel_load: operator %u reads tensor %d before it is written", k, o.inputs[i]);
            consumers[o.inputs[i]]++;
        }
        NNHIP_REQUIRE(ctx, producer[o.output] < 0 && (uint32_t)o.output != th.input_tensor, -EINVAL,
                      "kmodel_load: tensor %d is written twice", o.output);
        producer[o.output] = (int)k;
    }
    // conv -> byte table -> residual add chains collapse into the dense conv's epilogue
    std::vector<int> fused_add(th.n_ops, -1), fused_lut(th.n_ops, -1); // conv op -> add / table op folded into it
    std::vector<char> skipped(th.n_ops, 0);
    auto is_output = [&](int32_t t) { return (uint32_t)t >= th.output_tensor && (uint32_t)t < th.output_tensor + n_outputs; };
    auto dense_conv = [&](const hipf_op &c) {
        const bool depthwise = c.p[4] > 1 && c.p[1] == 1;
        return c.opcode == kOpConv2d && !depthwise && (int64_t)c.p[1] * c.p[4] > 4 && consumers[c.output] == 1 && !is_output(c.output);
    };
    for (uint32_t k = 1; k < th.n_ops; k++) {
        const hipf_op &lut = ops[k], &conv = ops[k - 1];
        if (lut.opcode == kOpLut && lut.n_inputs == 1 && lut.inputs[0] == conv.output && dense_conv(conv)) {
            fused_lut[k - 1] = (int)k;
            skipped[k] = 1;
        }
    }
    for (uint32_t k = 1; k < th.n_ops; k++) {
        const hipf_op &add = ops[k];
        if (add.opcode != kOpAdd || add.n_inputs != 2) continue;
        // the producer of the second operand: a dense conv, or a table already folded into one
        uint32_t c = k - 1;
        if (skipped[c] && ops[c].opcode == kOpLut && c >= 1 && fused_lut[c - 1] == (int)c) c--;
        const hipf_op &conv = ops[c];
        const int32_t produced = fused_lut[c] >= 0 ? ops[fused_lut[c]].output : conv.output;
        const bool ok_conv = fused_lut[c] >= 0 ? true : dense_conv(conv);
        if (conv.opcode == kOpConv2d && ok_conv && add.inputs[1] == produced && consumers[produced] == 1 && !is_output(produced) &&
            add.inputs[0] != produced && (fused_lut[c] >= 0 ? (uint32_t)fused_lut[c] == k - 1 : c == k - 1)) {
            fused_add[c] = (int)k;
            skipped[k] = 1;
        }
    }

    // 1x1 conv -> depthwise 3x3 -> 1x1 conv (+ the block's input), each consumed only by the next, on mid-sized
    // maps: one fused operator whose two expanded tensors never reach HBM (see nncase_hip_qblock)
    std::vector<char> block_head(th.n_ops, 0);
    auto pointwise = [&](const hipf_op &c) {
        return c.opcode == kOpConv2d && c.n_inputs == 1 && c.p[2] == 1 && c.p[3] == 1 && c.p[4] == 1 && c.p[5] == 1 && c.p[6] == 1 &&
               c.p[7] == 1 && c.p[8] == 1 && c.p[9] == 0 && c.p[10] == 0 && c.p[11] == 0 && c.p[12] == 0;
    };
    for (uint32_t k = 0; k + 2 < th.n_ops; k++) {
        const hipf_op &e = ops[k], &d = ops[k + 1], &pr = ops[k + 2];
        if (!pointwise(e) || !pointwise(pr) || d.opcode != kOpConv2d || d.n_inputs != 1) continue;
        const bool dw3 = d.p[1] == 1 && d.p[4] == d.p[0] && d.p[2] == 3 && d.p[3] == 3 && d.p[5] == d.p[6] && (d.p[5] == 1 || d.p[5] == 2) &&
                         d.p[7] == 1 && d.p[8] == 1 && (unsigned)d.p[9] <= 1 && (unsigned)d.p[10] <= 1 && (unsigned)d.p[11] <= 1 &&
                         (unsigned)d.p[12] <= 1;
        if (!dw3 || d.inputs[0] != e.output || pr.inputs[0] != d.output) continue;
        if (consumers[e.output] != 1 || consumers[d.output] != 1 || is_output(e.output) || is_output(d.output)) continue;
        if (fused_lut[k] >= 0 || fused_lut[k + 1] >= 0 || fused_lut[k + 2] >= 0 || fused_add[k] >= 0 || fused_add[k + 1] >= 0) continue;
        if (fused_add[k + 2] >= 0 && (ops[fused_add[k + 2]].inputs[0] != e.inputs[0] || d.p[5] != 1)) continue;
        nncase_hip_qblock_desc_t bd{};
        bd.in_channels = e.p[1], bd.mid_channels = e.p[0], bd.out_channels = pr.p[0];
        if (d.p[0] != e.p[0] || pr.p[1] != e.p[0] || !nncase_hip_qblock_supported(&bd)) continue;
        const hipf_tensor &te = m->tensors[e.output], &td = m->tensors[d.output];
        const uint64_t tiles7 = (uint64_t)((td.dims[1] + 6) / 7) * ((td.dims[2] + 6) / 7);
        // where it pays: mid-sized maps, at least 64 workgroups
        if (!((uint64_t)td.dims[1] * td.dims[2] >= 196 && (uint64_t)te.dims[1] * te.dims[2] <= 784 && td.dims[0] * tiles7 >= 64)) continue;
        block_head[k] = 1;
        skipped[k + 1] = skipped[k + 2] = 1;
        k += 2;
    }

    auto rd = [&](uint64_t off, size_t bytes) -> const uint8_t * {
        if (off == kNoRdata || off > rdata.n || bytes > rdata.n - off) return nullptr;
        return rdata.p + off;
    };

    // A dense conv whose result (behind its folded table / add) is read by one channel concat only writes its slice
    // of the concat's tensor itself.  The concat's requantisation of that input is a byte table: it is composed with
    // the conv's own table or becomes it; behind a folded add there is no table stage, so such a conv qualifies
    // only when that requantisation is the identity.  The concat then skips the input, and disappears when none is left.
    struct Through {
        int concat = -1, offset = 0, stride = 0;
        bool has_table = false;
        uint8_t table[256];
    };
    std::vector<Through> through(th.n_ops);
    {
        std::vector<int> owner(th.n_ops, -1); // folded table / add op -> its conv
        for (uint32_t k = 0; k < th.n_ops; k++) {
            if (fused_lut[k] >= 0) owner[fused_lut[k]] = (int)k;
            if (fused_add[k] >= 0) owner[fused_add[k]] = (int)k;
        }
        for (uint32_t ci = 0; ci < th.n_ops; ci++) {
            const hipf_op &cn = ops[ci];
            if (cn.opcode != kOpConcat || skipped[ci]) continue;
            const hipf_tensor &tc = m->tensors[cn.output];
            uint64_t total = 0;
            for (uint32_t i = 0; i < cn.n_inputs; i++) total += m->tensors[cn.inputs[i]].dims[3];
            if (tc.dtype != NNCASE_HIP_DT_U8 || total != tc.dims[3] || tc.scale == 0.f) continue; // (refused when it is recorded)
            int off = 0;
            for (uint32_t i = 0; i < cn.n_inputs; i++) {
                const int32_t t = cn.inputs[i];
                const hipf_tensor &tx = m->tensors[t];
                const int at = off;
                off += (int)tx.dims[3];
                const int p = producer[t];
                if (p < 0) continue;
                const int c = owner[p] >= 0 ? owner[p] : p;
                const hipf_op &conv = ops[c];
                const int last = fused_add[c] >= 0 ? fused_add[c] : fused_lut[c] >= 0 ? fused_lut[c] : c;
                if (conv.opcode != kOpConv2d || skipped[c] || block_head[c] || last != p || through[c].concat >= 0) continue;
                if (consumers[t] != 1 || is_output(t) || tx.dtype != NNCASE_HIP_DT_U8 || !dense_conv(conv)) continue;
                if (tx.dims[0] != tc.dims[0] || tx.dims[1] != tc.dims[1] || tx.dims[2] != tc.dims[2] || (uint32_t)conv.p[0] != tx.dims[3])
                    continue;
                uint8_t requant[256];
                if (nncase_hip_make_unary_lut(NNCASE_HIP_LUT_REQUANT, tqp((uint32_t)t), tqp((uint32_t)cn.output), requant) != 0) continue;
                bool identity = true;
                for (int v = 0; v < 256; v++) identity = identity && requant[v] == v;
                Through w;
                if (fused_add[c] >= 0) {
                    if (!identity) continue;
                } else if (fused_lut[c] >= 0) {
                    const uint8_t *own = rd(ops[fused_lut[c]].rdata0, 256);
                    if (!own) continue;
                    for (int v = 0; v < 256; v++) w.table[v] = requant[own[v]];
                    w.has_table = true;
                } else if (!identity) {
                    memcpy(w.table, requant, 256);
                    w.has_table = true;
                }
                w.concat = (int)ci, w.offset = at, w.stride = (int)tc.dims[3];
                through[c] = w;
            }
        }
    }

    // A Dequantize that alone reads a dense conv's result (behind its folded table / add) is done by that conv: it
    // stores the float32 value of its u8 result.
    std::vector<int> fused_deq(th.n_ops, -1); // conv op -> the dequantize op behind it
    for (uint32_t k = 0; k < th.n_ops; k++) {
        const hipf_op &dq = ops[k];
        if (dq.opcode != kOpDequantize || dq.n_inputs != 1) continue;
        const int32_t t = dq.inputs[0];
        const int p = producer[t];
        if (p < 0 || consumers[t] != 1 || is_output(t)) continue;
        int c = p;
        for (uint32_t q = 0; q < th.n_ops; q++)
            if (fused_lut[q] == p || fused_add[q] == p) c = (int)q;
        const hipf_op &conv = ops[c];
        const int last = fused_add[c] >= 0 ? fused_add[c] : fused_lut[c] >= 0 ? fused_lut[c] : c;
        if (conv.opcode != kOpConv2d || skipped[c] || block_head[c] || last != p || through[c].concat >= 0 || !dense_conv(conv)) continue;
        if (m->tensors[t].dtype != NNCASE_HIP_DT_U8 || m->tensors[dq.output].dtype != NNCASE_HIP_DT_F32 ||
            elems((uint32_t)t) != elems((uint32_t)dq.output))
            continue;
        fused_deq[c] = (int)k;
        skipped[k] = 1;
    }

    // A float32 -> u8 quantize read only by a channel padding is done by that operator (quantize and pack in one pass).
    std::vector<int> fused_quant(th.n_ops, -1); // pad_channels op -> the quantize op in front of it
    for (uint32_t k = 0; k < th.n_ops; k++) {
        if (ops[k].opcode != kOpPadChannels || ops[k].n_inputs != 1) continue;
        const int32_t t = ops[k].inputs[0];
        const int q = producer[t];
        if (q < 0 || ops[q].opcode != kOpQuantize || ops[q].n_inputs != 1 || consumers[t] != 1 || is_output(t)) continue;
        if (m->tensors[ops[q].inputs[0]].dtype != NNCASE_HIP_DT_F32 || m->tensors[t].dtype != NNCASE_HIP_DT_U8 || m->tensors[t].scale == 0.f ||
            m->tensors[t].dims[3] > 4 || elems((uint32_t)ops[q].inputs[0]) != elems((uint32_t)t))
            continue;
        const hipf_tensor &tp = m->tensors[ops[k].output], &tq = m->tensors[t];
        const bool plain = tp.dims[3] == 4 && tp.dims[1] == tq.dims[1] && tp.dims[2] == tq.dims[2];
        const bool blocks = tp.dims[3] == 16 && tq.dims[1] == 2 * tp.dims[1] && tq.dims[2] == 2 * tp.dims[2];
        if (tp.dtype != NNCASE_HIP_DT_U8 || !(plain || blocks)) continue;
        fused_quant[k] = q;
        skipped[q] = 1;
    }

    // A dense 1x1 convolution (behind its folded table / add) that a second dense 1x1 convolution reads runs with it as
    // one launch where the two are latency-bound (see nncase_hip_qpointwise_pair): while the weight bytes the pair's
    // workgroups stream between them and their number stay small.  A 3x3 depthwise convolution that only the first of
    // them reads joins the launch while it has few channels.
    std::vector<int> pair_second(th.n_ops, -1), pair_front(th.n_ops, -1);
    {
        constexpr uint64_t kStreamLimit = 4u << 20, kMaxPixelTiles = 1024;
        constexpr int kFrontMaxChannels = 256;
        auto plain_pointwise = [&](uint32_t k) {
            return pointwise(ops[k]) && !skipped[k] && !block_head[k] && through[k].concat < 0 && fused_deq[k] < 0 &&
                   m->tensors[ops[k].output].dtype == NNCASE_HIP_DT_U8 && m->tensors[ops[k].inputs[0]].dtype == NNCASE_HIP_DT_U8;
        };
        for (uint32_t k = 0; k < th.n_ops; k++) {
            if (!plain_pointwise(k)) continue;
            const int tail = fused_add[k] >= 0 ? fused_add[k] : fused_lut[k] >= 0 ? fused_lut[k] : (int)k;
            const int32_t mid = ops[tail].output;
            int j = -1;
            for (uint32_t q = (uint32_t)tail + 1; q < th.n_ops && j < 0; q++)
                if (plain_pointwise(q) && ops[q].inputs[0] == mid && fused_add[q] < 0) j = (int)q;
            if (j < 0) continue;
            const int k1 = ops[k].p[1], n1 = ops[k].p[0], n2 = ops[j].p[0];
            if (ops[j].p[1] != n1 || !nncase_hip_qpointwise_pair_supported(k1, n1, n2)) continue;
            const hipf_tensor &tm = m->tensors[mid];
            const uint64_t ptiles = ((uint64_t)tm.dims[0] * tm.dims[1] * tm.dims[2] + 15) / 16;
            if (ptiles > kMaxPixelTiles || ptiles * ((uint64_t)k1 * n1 + (uint64_t)n1 * n2) > kStreamLimit) continue;
            pair_second[k] = j;
            skipped[j] = 1;
            const int32_t x = ops[k].inputs[0];
            const int d = producer[x];
            if (d < 0 || skipped[d] || k1 > kFrontMaxChannels) continue;
            const hipf_op &dc = ops[d];
            const bool dw3 = dc.opcode == kOpConv2d && dc.n_inputs == 1 && dc.p[1] == 1 && dc.p[4] == dc.p[0] && dc.p[0] == k1 && dc.p[2] == 3 &&
                             dc.p[3] == 3 && dc.p[5] == dc.p[6] && (dc.p[5] == 1 || dc.p[5] == 2) && dc.p[7] == 1 && dc.p[8] == 1;
            if (!dw3 || consumers[x] != 1 || is_output(x) || m->tensors[x].dtype != NNCASE_HIP_DT_U8) continue;
            pair_front[k] = d;
            skipped[d] = 1;
        }
    }

    // A global average pool read by one dense 1x1 convolution alone (a classifier's tail) is computed by that
    // convolution's launch where that pays: a few rows (see nncase_hip_qglobal_avgpool_qconv2d).
    std::vector<int> pool_reader(th.n_ops, -1), pool_of(th.n_ops, -1); // pool op -> conv op and back
    for (uint32_t k = 0; k < th.n_ops; k++) {
        const hipf_op &g = ops[k];
        if (g.opcode != kOpGlobalAvgPool || g.n_inputs != 1 || skipped[k] || consumers[g.output] != 1 || is_output(g.output)) continue;
        const hipf_tensor &tg = m->tensors[g.inputs[0]], &tp = m->tensors[g.output];
        if (tg.dtype != NNCASE_HIP_DT_U8 || tp.dtype != NNCASE_HIP_DT_U8 || tp.dims[0] != tg.dims[0] || tp.dims[3] != tg.dims[3] || tp.dims[1] != 1 ||
            tp.dims[2] != 1)
            continue;
        for (uint32_t c = k + 1; c < th.n_ops; c++) {
            if (ops[c].n_inputs != 1 || ops[c].inputs[0] != g.output) continue;
            // (the conditions of nncase_hip_qglobal_avgpool_qconv2d_supported, decided here because the pooled tensor gets no buffer)
            const hipf_tensor &ty = m->tensors[ops[c].output];
            if (pointwise(ops[c]) && !skipped[c] && !block_head[c] && through[c].concat < 0 && fused_add[c] < 0 && pair_second[c] < 0 &&
                (ty.dtype == NNCASE_HIP_DT_U8 || fused_deq[c] >= 0) && rows_shapes_ok(ops[c].p[1], ops[c].p[0], (int64_t)tp.dims[0]) &&
                pool_front_pays((int)tg.dims[0], (int)(tg.dims[1] * tg.dims[2]), (int)tg.dims[3]))
                pool_reader[k] = (int)c, pool_of[c] = (int)k;
            break;
        }
    }

    // ---- device buffers ---------------------------------------------------------------------------
    m->buffers.assign(th.n_tensors, nullptr);
    m->owns.assign(th.n_tensors, 0);
    for (uint32_t k = 0; k < th.n_ops; k++) { // tensors that only exist inside a fused operator
        if (fused_add[k] >= 0 || fused_lut[k] >= 0) m->owns[ops[k].output] = 2;
        if (fused_add[k] >= 0 && fused_lut[k] >= 0) m->owns[ops[fused_lut[k]].output] = 2;
        if (block_head[k]) m->owns[ops[k].output] = m->owns[ops[k + 1].output] = 2;
        if (pair_front[k] >= 0) m->owns[ops[pair_front[k]].output] = 2; // computed inside the pair's launch
        if (pool_reader[k] >= 0) m->owns[ops[k].output] = 2;            // ... inside the convolution's
        if (fused_quant[k] >= 0) m->owns[ops[fused_quant[k]].output] = 2;
        if (fused_deq[k] >= 0) { // the u8 result is never stored
            m->owns[ops[k].output] = 2;
            if (fused_lut[k] >= 0) m->owns[ops[fused_lut[k]].output] = 2;
            if (fused_add[k] >= 0) m->owns[ops[fused_add[k]].output] = 2;
        }
        if (through[k].concat >= 0) { // no tensor of its own: the bytes live in the concat's tensor
            m->owns[ops[k].output] = 2;
            if (fused_lut[k] >= 0) m->owns[ops[fused_lut[k]].output] = 2;
            if (fused_add[k] >= 0) m->owns[ops[fused_add[k]].output] = 2;
        }
    }
    for (uint32_t k = 0; k < th.n_ops; k++) // a reshaped tensor is its input's buffer under other extents
        if (ops[k].opcode == kOpReshape && !skipped[k]) m->owns[ops[k].output] = 2;
    for (uint32_t t = 0; t < th.n_tensors; t++) {
        if (m->owns[t] == 2) {
            m->owns[t] = 0;
            continue;
        }
        NNHIP_HIP(ctx, hipMalloc(&m->buffers[t], elems(t) * dtype_size(m->tensors[t].dtype)));
        m->owns[t] = 1;
    }

    // ---- operators ----------------------------------------------------------------------------------
    NNHIP_REQUIRE(ctx, nncase_hip_function_create(ctx, &m->fn) == 0, -ENOMEM, "kmodel_load: cannot create the function");
    // Everything a convolution operator needs short of recording it: checks, packed weights (kept in m->weights), the
    // arguments with whatever is folded into the epilogue, and where the result goes.
    auto prepare_conv = [&](uint32_t k, nncase_hip_weights_t **wt_out, nncase_hip_conv2d_args_t *a_out, void **y_out,
                            const uint8_t **w_host) -> int {
        const hipf_op &o = ops[k];
        const uint32_t in0 = (uint32_t)o.inputs[0], dst = (uint32_t)o.output;
        const hipf_tensor &ti = m->tensors[in0], &to = m->tensors[dst];
        int rc = -EINVAL;
        const int oc = o.p[0], gic = o.p[1], kh = o.p[2], kw = o.p[3], groups = o.p[4];
        NNHIP_REQUIRE(ctx, oc > 0 && gic > 0 && kh > 0 && kw > 0 && groups > 0, -EINVAL, "kmodel_load: op %u conv shape", k);
        // a convolution whose Quantize consumer is absent writes float32 (the matmul of config 1 is one)
        NNHIP_REQUIRE(ctx, ti.dtype == NNCASE_HIP_DT_U8 && (to.dtype == NNCASE_HIP_DT_U8 || to.dtype == NNCASE_HIP_DT_F32),
                      -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "kmodel_load: op %u conv needs a u8 input and a u8 or f32 output", k);
        NNHIP_REQUIRE(ctx, to.dtype == NNCASE_HIP_DT_U8 || (fused_lut[k] < 0 && fused_add[k] < 0), -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                      "kmodel_load: op %u writes f32, which a byte table or a residual add cannot follow", k);
        NNHIP_REQUIRE(ctx, (uint32_t)(gic * groups) == ti.dims[3] && (uint32_t)oc == to.dims[3] && ti.dims[0] == to.dims[0],
                      -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u conv channels / batch do not match its tensors", k);
        const size_t wbytes = (size_t)oc * gic * kh * kw;
        const uint8_t *w = rd(o.rdata0, wbytes);
        NNHIP_REQUIRE(ctx, w, -EINVAL, "kmodel_load: op %u weights outside .rdata", k);
        const uint8_t *b = nullptr;
        if (o.rdata1 != kNoRdata) {
            b = rd(o.rdata1, (size_t)oc * 4);
            NNHIP_REQUIRE(ctx, b && (o.rdata1 & 3) == 0, -EINVAL, "kmodel_load: op %u bias outside .rdata or misaligned", k);
        }
        nncase_hip_conv2d_desc_t desc{};
        desc.in_channels = gic * groups, desc.out_channels = oc, desc.kernel_h = kh, desc.kernel_w = kw, desc.groups = groups;
        desc.w_qp = nncase_hip_quant_param_t{o.p[13], o.f[2]};
        desc.expected_pixels = (int64_t)to.dims[0] * to.dims[1] * to.dims[2];
        nncase_hip_weights_t *wt = nullptr;
        rc = nncase_hip_qconv2d_prepack(ctx, &desc, w, reinterpret_cast<const int32_t *>(b), &wt);
        if (rc) return rc;
        m->weights.push_back(wt);
        nncase_hip_conv2d_args_t a{};
        a.batch = (int)ti.dims[0], a.in_h = (int)ti.dims[1], a.in_w = (int)ti.dims[2];
        a.stride_h = o.p[5], a.stride_w = o.p[6], a.dilation_h = o.p[7], a.dilation_w = o.p[8];
        a.pad_h_before = o.p[9], a.pad_h_after = o.p[10], a.pad_w_before = o.p[11], a.pad_w_after = o.p[12];
        a.x_qp = tqp(in0), a.y_qp = tqp(dst);
        a.clamp_min = o.f[0], a.clamp_max = o.f[1];
        a.out_dtype = (int32_t)to.dtype;
        NNHIP_REQUIRE(ctx, windowed_output_size(a.in_h, kh, a.stride_h, a.dilation_h, a.pad_h_before, a.pad_h_after) == (int)to.dims[1] &&
                               windowed_output_size(a.in_w, kw, a.stride_w, a.dilation_w, a.pad_w_before, a.pad_w_after) == (int)to.dims[2],
                      -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u conv output extent does not match its tensor", k);
        void *y = m->buffers[dst];
        if (fused_lut[k] >= 0) {
            const hipf_op &lut = ops[fused_lut[k]];
            const uint8_t *table = rd(lut.rdata0, 256);
            NNHIP_REQUIRE(ctx, table, -EINVAL, "kmodel_load: op %d table outside .rdata", fused_lut[k]);
            NNHIP_REQUIRE(ctx, elems((uint32_t)lut.output) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                          "kmodel_load: op %d shapes differ", fused_lut[k]);
            // (a conv that writes into its concat applies its table and the concat's requantisation in one)
            rc = through[k].has_table ? nncase_hip_weights_set_post_lut(ctx, wt, through[k].table, tqp((uint32_t)ops[through[k].concat].output))
                                      : nncase_hip_weights_set_post_lut(ctx, wt, table, tqp((uint32_t)lut.output));
            if (rc) return rc;
            y = m->buffers[lut.output];
        } else if (through[k].has_table) {
            rc = nncase_hip_weights_set_post_lut(ctx, wt, through[k].table, tqp((uint32_t)ops[through[k].concat].output));
            if (rc) return rc;
        }
        if (fused_add[k] >= 0) {
            const hipf_op &add = ops[fused_add[k]];
            const uint32_t res = (uint32_t)add.inputs[0], sum = (uint32_t)add.output;
            NNHIP_REQUIRE(ctx, elems(res) == elems(dst) && elems(sum) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                          "kmodel_load: op %d add shapes differ", fused_add[k]);
            a.residual_dev = static_cast<const uint8_t *>(m->buffers[res]);
            a.residual_qp = tqp(res), a.sum_qp = tqp(sum);
            a.sum_clamp_min = add.f[0], a.sum_clamp_max = add.f[1];
            y = m->buffers[sum];
        }
        if (fused_deq[k] >= 0) {
            y = m->buffers[ops[fused_deq[k]].output];
            a.out_dtype = NNCASE_HIP_DT_F32, a.dequantize_output = 1;
        }
        if (through[k].concat >= 0) {
            y = m->buffers[ops[through[k].concat].output];
            a.out_channel_stride = through[k].stride, a.out_channel_offset = through[k].offset;
        }
        *wt_out = wt, *a_out = a, *y_out = y, *w_host = w;
        return 0;
    };

    for (uint32_t k = 0; k < th.n_ops; k++) {
        if (skipped[k]) continue;
        const hipf_op &o = ops[k];
        const uint32_t in0 = (uint32_t)o.inputs[0], dst = (uint32_t)o.output;
        const hipf_tensor &ti = m->tensors[in0], &to = m->tensors[dst];
        int rc = -EINVAL;
        if (block_head[k]) {
            const hipf_op &d = ops[k + 1], &pr = ops[k + 2];
            const uint32_t te = (uint32_t)o.output, td = (uint32_t)d.output, tp = (uint32_t)pr.output;
            const int cin = o.p[1], mid = o.p[0], cout = pr.p[0];
            NNHIP_REQUIRE(ctx, ti.dtype == NNCASE_HIP_DT_U8 && m->tensors[tp].dtype == NNCASE_HIP_DT_U8 && (uint32_t)cin == ti.dims[3] &&
                                   (uint32_t)cout == m->tensors[tp].dims[3] && ti.dims[0] == m->tensors[tp].dims[0],
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u block channels / batch do not match its tensors", k);
            const uint8_t *wgt[3] = {rd(o.rdata0, (size_t)mid * cin), rd(d.rdata0, (size_t)mid * 9), rd(pr.rdata0, (size_t)cout * mid)};
            const int32_t *bia[3] = {nullptr, nullptr, nullptr};
            const hipf_op *stage[3] = {&o, &d, &pr};
            for (int i = 0; i < 3; i++) {
                NNHIP_REQUIRE(ctx, wgt[i], -EINVAL, "kmodel_load: op %u weights outside .rdata", k + i);
                if (stage[i]->rdata1 != kNoRdata) {
                    const uint8_t *b = rd(stage[i]->rdata1, (size_t)stage[i]->p[0] * 4);
                    NNHIP_REQUIRE(ctx, b && (stage[i]->rdata1 & 3) == 0, -EINVAL, "kmodel_load: op %u bias outside .rdata or misaligned", k + i);
                    bia[i] = reinterpret_cast<const int32_t *>(b);
                }
            }
            nncase_hip_qblock_desc_t bd{};
            bd.in_channels = cin, bd.mid_channels = mid, bd.out_channels = cout;
            bd.expand_w_qp = nncase_hip_quant_param_t{o.p[13], o.f[2]};
            bd.dw_w_qp = nncase_hip_quant_param_t{d.p[13], d.f[2]};
            bd.project_w_qp = nncase_hip_quant_param_t{pr.p[13], pr.f[2]};
            nncase_hip_qblock_t *blk = nullptr;
            rc = nncase_hip_qblock_prepack(ctx, &bd, wgt[0], bia[0], wgt[1], bia[1], wgt[2], bia[2], &blk);
            if (rc) return rc;
            m->blocks.push_back(blk);
            nncase_hip_qblock_args_t a{};
            a.batch = (int)ti.dims[0], a.in_h = (int)ti.dims[1], a.in_w = (int)ti.dims[2], a.stride = d.p[5];
            a.pad_h_before = d.p[9], a.pad_h_after = d.p[10], a.pad_w_before = d.p[11], a.pad_w_after = d.p[12];
            a.x_qp = tqp(in0), a.expand_qp = tqp(te), a.dw_qp = tqp(td), a.y_qp = tqp(tp);
            a.expand_clamp_min = o.f[0], a.expand_clamp_max = o.f[1];
            a.dw_clamp_min = d.f[0], a.dw_clamp_max = d.f[1];
            a.clamp_min = pr.f[0], a.clamp_max = pr.f[1];
            NNHIP_REQUIRE(ctx, m->tensors[te].dims[1] == ti.dims[1] && m->tensors[te].dims[2] == ti.dims[2] &&
                                   windowed_output_size(a.in_h, 3, a.stride, 1, a.pad_h_before, a.pad_h_after) == (int)m->tensors[tp].dims[1] &&
                                   windowed_output_size(a.in_w, 3, a.stride, 1, a.pad_w_before, a.pad_w_after) == (int)m->tensors[tp].dims[2] &&
                                   m->tensors[td].dims[1] == m->tensors[tp].dims[1] && m->tensors[td].dims[2] == m->tensors[tp].dims[2],
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u block extents do not match its tensors", k);
            void *y = m->buffers[tp];
            if (fused_add[k + 2] >= 0) {
                const hipf_op &add = ops[fused_add[k + 2]];
                const uint32_t sum = (uint32_t)add.output;
                NNHIP_REQUIRE(ctx, elems(sum) == elems(tp) && elems(in0) == elems(tp), -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                              "kmodel_load: op %d add shapes differ", fused_add[k + 2]);
                a.add_input = 1;
                a.sum_qp = tqp(sum);
                a.sum_clamp_min = add.f[0], a.sum_clamp_max = add.f[1];
                y = m->buffers[sum];
            }
            rc = nncase_hip_function_add_qblock(m->fn, static_cast<const uint8_t *>(m->buffers[in0]), blk, static_cast<uint8_t *>(y), &a);
            if (rc) return rc;
            continue;
        }
        switch (o.opcode) {
        case kOpQuantize:
            NNHIP_REQUIRE(ctx, elems(in0) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u shapes differ", k);
            rc = nncase_hip_function_add_quantize(m->fn, m->buffers[in0], (int)ti.dtype, m->buffers[dst], (int)to.dtype, elems(dst),
                                                  tqp(dst));
            break;
        case kOpDequantize:
            NNHIP_REQUIRE(ctx, elems(in0) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u shapes differ", k);
            rc = nncase_hip_function_add_dequantize(m->fn, m->buffers[in0], (int)ti.dtype, m->buffers[dst], (int)to.dtype,
                                                    elems(dst), tqp(in0));
            break;
        case kOpConv2d: {
            nncase_hip_weights_t *wt = nullptr;
            nncase_hip_conv2d_args_t a{};
            void *y = nullptr;
            const uint8_t *w_host = nullptr;
            rc = prepare_conv(k, &wt, &a, &y, &w_host);
            if (rc) return rc;
            if (pool_of[k] >= 0) {
                // a global average pool that only this convolution reads: one launch for both where the library says it
                // pays (a few rows), else the pool now, in front of the convolution
                const hipf_op &g = ops[pool_of[k]];
                const uint32_t gin = (uint32_t)g.inputs[0];
                const hipf_tensor &tg = m->tensors[gin];
                NNHIP_REQUIRE(ctx, nncase_hip_qglobal_avgpool_qconv2d_supported(wt, &a, (int)tg.dims[1], (int)tg.dims[2]), -EINVAL,
                              "kmodel_load: op %u was planned as a pooled convolution and does not qualify", k);
                rc = nncase_hip_function_add_qglobal_avgpool_qconv2d(m->fn, static_cast<const uint8_t *>(m->buffers[gin]), (int)tg.dims[1],
                                                                     (int)tg.dims[2], tqp(gin), wt, y, &a);
                break;
            }
            if (pair_second[k] >= 0) {
                nncase_hip_weights_t *wt2 = nullptr, *wt0 = nullptr;
                nncase_hip_conv2d_args_t a2{}, a0{};
                void *y2 = nullptr, *y0 = nullptr;
                const uint8_t *w2_host = nullptr, *w0_host = nullptr;
                rc = prepare_conv((uint32_t)pair_second[k], &wt2, &a2, &y2, &w2_host);
                if (rc) return rc;
                nncase_hip_qpair_t *pr = nullptr;
                rc = nncase_hip_qpointwise_pair_create(ctx, wt, w_host, wt2, w2_host, &pr);
                if (rc) return rc;
                m->pairs.push_back(pr);
                if (pair_front[k] >= 0) {
                    rc = prepare_conv((uint32_t)pair_front[k], &wt0, &a0, &y0, &w0_host);
                    if (rc) return rc;
                    const void *x0 = m->buffers[ops[pair_front[k]].inputs[0]];
                    rc = nncase_hip_function_add_qdepthwise_pointwise_pair(m->fn, static_cast<const uint8_t *>(x0), wt0, &a0, pr,
                                                                           static_cast<uint8_t *>(y), static_cast<uint8_t *>(y2), &a, &a2);
                } else {
                    rc = nncase_hip_function_add_qpointwise_pair(m->fn, static_cast<const uint8_t *>(m->buffers[in0]), pr, static_cast<uint8_t *>(y),
                                                                 static_cast<uint8_t *>(y2), &a, &a2);
                }
                break;
            }
            rc = nncase_hip_function_add_qconv2d(m->fn, static_cast<const uint8_t *>(m->buffers[in0]), wt, y, &a);
            break;
        }
        case kOpAdd: {
            NNHIP_REQUIRE(ctx, o.n_inputs == 2, -EINVAL, "kmodel_load: op %u add needs two inputs", k);
            const uint32_t in1 = (uint32_t)o.inputs[1];
            NNHIP_REQUIRE(ctx, elems(in0) == elems(dst) && elems(in1) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                          "kmodel_load: op %u add shapes differ", k);
            rc = nncase_hip_function_add_qadd(m->fn, static_cast<const uint8_t *>(m->buffers[in0]), tqp(in0),
                                              static_cast<const uint8_t *>(m->buffers[in1]), tqp(in1),
                                              static_cast<uint8_t *>(m->buffers[dst]), tqp(dst), o.f[0], o.f[1], elems(dst));
            break;
        }
        case kOpGlobalAvgPool:
            NNHIP_REQUIRE(ctx, to.dims[0] == ti.dims[0] && to.dims[3] == ti.dims[3] && to.dims[1] == 1 && to.dims[2] == 1,
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u pool shapes", k);
            if (pool_reader[k] >= 0) { // recorded with the convolution that alone reads it
                rc = 0;
                break;
            }
            rc = nncase_hip_function_add_qglobal_avgpool(m->fn, static_cast<const uint8_t *>(m->buffers[in0]),
                                                         static_cast<uint8_t *>(m->buffers[dst]), (int)ti.dims[0], (int)ti.dims[1],
                                                         (int)ti.dims[2], (int)ti.dims[3], tqp(in0), tqp(dst));
            break;
        case kOpLut: {
            const uint8_t *lut = rd(o.rdata0, 256);
            NNHIP_REQUIRE(ctx, lut, -EINVAL, "kmodel_load: op %u table outside .rdata", k);
            NNHIP_REQUIRE(ctx, elems(in0) == elems(dst), -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u shapes differ", k);
            rc = nncase_hip_function_add_lut_u8(m->fn, static_cast<const uint8_t *>(m->buffers[in0]),
                                                static_cast<uint8_t *>(m->buffers[dst]), elems(dst), lut);
            break;
        }
        case kOpConcat: {
            const uint8_t *ins[8];
            int32_t ch[8];
            nncase_hip_quant_param_t qps[8];
            uint32_t total = 0, to_copy = 0;
            for (uint32_t i = 0; i < o.n_inputs; i++) {
                const hipf_tensor &x = m->tensors[o.inputs[i]];
                NNHIP_REQUIRE(ctx, x.dims[0] == to.dims[0] && x.dims[1] == to.dims[1] && x.dims[2] == to.dims[2],
                              -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u concat input %u extent", k, i);
                ins[i] = static_cast<const uint8_t *>(m->buffers[o.inputs[i]]); // null: written in place by its conv
                to_copy += ins[i] != nullptr;
                ch[i] = (int32_t)x.dims[3];
                qps[i] = tqp((uint32_t)o.inputs[i]);
                total += x.dims[3];
            }
            NNHIP_REQUIRE(ctx, total == to.dims[3], -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u concat channels", k);
            if (to_copy == 0) { // every slice is written by its producer
                rc = 0;
                break;
            }
            rc = nncase_hip_function_add_qconcat_channels(m->fn, (int32_t)o.n_inputs, ins, ch, qps, static_cast<uint8_t *>(m->buffers[dst]),
                                                          tqp(dst), (int64_t)to.dims[0] * to.dims[1] * to.dims[2]);
            break;
        }
        case kOpResizeNearest:
            NNHIP_REQUIRE(ctx, ti.dtype == to.dtype && ti.dims[0] == to.dims[0] && ti.dims[3] == to.dims[3],
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u resize tensors", k);
            rc = nncase_hip_function_add_resize_nearest(m->fn, m->buffers[in0], m->buffers[dst], (int)dtype_size(ti.dtype),
                                                        (int)ti.dims[0], (int)ti.dims[1], (int)ti.dims[2], (int)ti.dims[3],
                                                        (int)to.dims[1], (int)to.dims[2], o.p[0], o.p[1]);
            break;
        case kOpMaxPool:
            NNHIP_REQUIRE(ctx, ti.dims[0] == to.dims[0] && ti.dims[3] == to.dims[3] && o.p[0] > 0 && o.p[1] > 0 && o.p[2] >= 0 &&
                                   windowed_output_size((int)ti.dims[1], o.p[0], o.p[1], 1, o.p[2], o.p[2]) == (int)to.dims[1] &&
                                   windowed_output_size((int)ti.dims[2], o.p[0], o.p[1], 1, o.p[2], o.p[2]) == (int)to.dims[2],
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u pool tensors", k);
            rc = nncase_hip_function_add_qmaxpool2d(m->fn, static_cast<const uint8_t *>(m->buffers[in0]),
                                                    static_cast<uint8_t *>(m->buffers[dst]), (int)ti.dims[0], (int)ti.dims[1],
                                                    (int)ti.dims[2], (int)ti.dims[3], o.p[0], o.p[0], o.p[1], o.p[1], o.p[2], o.p[2],
                                                    o.p[2], o.p[2], tqp(in0), tqp(dst));
            break;
        case kOpLayout:
            // p[0] = 0: the input holds N, C, H, W in that order and the output is channels-last; 1: the reverse
            // (both tensor records give their extents as N, H, W, C)
            NNHIP_REQUIRE(ctx, ti.dtype == to.dtype && memcmp(ti.dims, to.dims, sizeof(ti.dims)) == 0 && (o.p[0] == 0 || o.p[0] == 1),
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u layout tensors / direction", k);
            rc = nncase_hip_function_add_layout(m->fn, m->buffers[in0], m->buffers[dst], (int)dtype_size(ti.dtype), (int)ti.dims[0],
                                                (int)ti.dims[3], (int)ti.dims[1], (int)ti.dims[2], o.p[0]);
            break;
        case kOpReshape:
            NNHIP_REQUIRE(ctx, ti.dtype == to.dtype && elems(in0) == elems(dst) && m->buffers[in0] && !is_output((int32_t)dst),
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u reshapes %zu elements into %zu", k, elems(in0), elems(dst));
            m->buffers[dst] = m->buffers[in0];
            rc = 0;
            break;
        case kOpPadChannels: {
            // channels padded to 4, and with halved extents 2 x 2 blocks of such pixels as 16-channel pixels
            const bool blocks = to.dims[3] == 16 && ti.dims[1] == 2 * to.dims[1] && ti.dims[2] == 2 * to.dims[2];
            NNHIP_REQUIRE(ctx, ti.dtype == to.dtype && ti.dims[0] == to.dims[0] && ti.dims[3] <= to.dims[3] &&
                                   (blocks ? ti.dims[3] <= 4 : ti.dims[1] == to.dims[1] && ti.dims[2] == to.dims[2]),
                          -NNCASE_HIP_ERR_SHAPE_MISMATCH, "kmodel_load: op %u channel padding tensors", k);
            const int32_t shape[4] = {(int32_t)ti.dims[0], (int32_t)ti.dims[1], (int32_t)ti.dims[2], (int32_t)ti.dims[3]};
            const int32_t axes[3] = {1, 2, 3}, lanes[3] = {2, 2, 4}, lanes_c = (int32_t)to.dims[3];
            const int32_t n_axes = blocks ? 3 : 1;
            const int32_t *ax = blocks ? axes : axes + 2, *ln = blocks ? lanes : &lanes_c;
            if (fused_quant[k] >= 0) {
                const uint32_t src = (uint32_t)ops[fused_quant[k]].inputs[0];
                rc = nncase_hip_function_add_quantize_pack(m->fn, static_cast<const float *>(m->buffers[src]),
                                                           static_cast<uint8_t *>(m->buffers[dst]), 4, shape, n_axes, ax, ln, tqp(in0));
            } else {
                rc = nncase_hip_function_add_pack(m->fn, m->buffers[in0], m->buffers[dst], (int)dtype_size(ti.dtype), 4, shape, n_axes, ax, ln);
            }
            break;
        }
        default:
            return fail(ctx, -NNCASE_HIP_ERR_RUNTIME_NOT_FOUND, "kmodel_load: operator %u has unknown opcode %u", k, o.opcode);
        }
        if (rc) return rc;
    }
    *out = m.release();
    return 0;
}

extern "C" int nncase_hip_kmodel_function(nncase_hip_kmodel_t *m, nncase_hip_function_t **fn) {
    if (!m || !fn) return -EINVAL;
    *fn = m->fn;
    return 0;
}

extern "C" int nncase_hip_kmodel_tensor(nncase_hip_kmodel_t *m, int32_t which, void **dev_ptr, int32_t *dtype, int32_t *dims4) {
    if (!m) return -EINVAL;
    uint32_t t;
    if (which == NNCASE_HIP_KMODEL_INPUT) t = m->input_tensor;
    else if (which <= NNCASE_HIP_KMODEL_OUTPUT && (uint32_t)(NNCASE_HIP_KMODEL_OUTPUT - which) < m->n_outputs)
        t = m->output_tensor + (uint32_t)(NNCASE_HIP_KMODEL_OUTPUT - which);
    else if (which >= 0 && (size_t)which < m->tensors.size()) t = (uint32_t)which;
    else return fail(m->ctx, -EINVAL, "kmodel_tensor: index %d out of range", which);
    if (dev_ptr) *dev_ptr = m->buffers[t]; // null for a tensor that only exists inside a fused operator
    if (dtype) *dtype = (int32_t)m->tensors[t].dtype;
    if (dims4)
        for (int i = 0; i < 4; i++) dims4[i] = (int32_t)m->tensors[t].dims[i];
    return 0;
}
