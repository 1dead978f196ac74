"""GPU: kmodel files written by nncase_amd.kmodel and loaded by the native loader give the oracle's
bytes; malformed files are refused with the reference's error codes."""
import json
import os
import struct

import numpy as np
import pytest

from nncase_amd import kmodel as km
from nncase_amd import netbuilder as nb
from nncase_amd import runtime as rt
from oracle import netref

pytestmark = pytest.mark.gpu
f32 = np.float32
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def run_and_check(hip_ctx, qg, x, stackvm_main=False):
    data = km.compile_quant_graph(qg, x.shape[0], stackvm_main=stackvm_main)
    model = rt.LoadedKModel(hip_ctx, data)
    assert model.input_shape == x.shape and model.input_dtype == np.float32
    y = model.run(x)
    want, outs = netref.run_integer(qg, x, keep_all=True)
    want_nhwc = np.ascontiguousarray(np.asarray(want).transpose(0, 2, 3, 1)) if np.asarray(want).ndim == 4 else want
    assert np.array_equal(y.reshape(want_nhwc.shape).view(np.uint32), want_nhwc.view(np.uint32))
    # every tensor the loader materialised holds the oracle's bytes (tensor i + 1 is node i)
    fused = 0
    for i, ref in enumerate(outs):
        buf, shape, dtype = model.tensor(i + 1)
        if buf is None:
            fused += 1
            continue
        got = buf.download(shape, dtype).transpose(0, 3, 1, 2)
        assert np.array_equal(got, ref), f"node {i} ({qg.nodes[i].name})"
    return model, y, fused


def test_conv_block_kmodel(hip_ctx):
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((8, 56, 56, 64), dtype=f32))
    x = rng.random((2, 56, 56, 64), dtype=f32)
    model, y, fused = run_and_check(hip_ctx, qg, x)
    assert fused == 1 and len(model.fn) == 4             # (the last conv stores the dequantised output itself)
    model.fn.capture()                                   # the loaded function replays as a HIP graph
    for _ in range(2):
        assert np.array_equal(model.run(x).view(np.uint32), y.view(np.uint32))
    with pytest.raises(rt.HipError) as e:
        model.run(x[:1])
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH


@pytest.mark.parametrize("batch", [4, 1])
def test_mobilenetv2_kmodel(hip_ctx, batch):
    rng = np.random.default_rng(3)
    qg = nb.quantize_graph(nb.mobilenet_v2(seed=2), rng.random((8, 224, 224, 3), dtype=f32))
    x = rng.random((batch, 224, 224, 3), dtype=f32)
    model, y, fused = run_and_check(hip_ctx, qg, x)
    ref = nb.HipModel(hip_ctx, qg, batch, capture_graph=False)
    assert np.array_equal(ref.run(x).view(np.uint32).ravel(), y.view(np.uint32).ravel())
    # the loader folds what HipModel folds: the ten residual adds, the input's quantize into the pack in front of the stem,
    # the output's dequantize into the classifier; at batch 4 the two 28x28 blocks (64 workgroups each) whole and the
    # projection -> expansion pairs of the 14x14 and 7x7 maps; at batch 1 every such pair, seven of them with
    # their depthwise convolution in front
    assert len(model.fn) == len(ref.fn) == {4: 43, 1: 30}[batch]
    assert fused == len(ref.never_written)
    kernels = [model.fn.op_kernel(i) for i in range(len(model.fn))]
    assert kernels == [ref.fn.op_kernel(i) for i in range(len(ref.fn))]
    assert kernels.count("dw3x3+qpointwise_pair_kernel") == len(ref.pair_fronts) == {4: 1, 1: 7}[batch]


def test_malformed_files_are_refused(hip_ctx):
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((2, 56, 56, 64), dtype=f32))
    good = km.compile_quant_graph(qg, 1)

    def code(data):
        with pytest.raises(rt.HipError) as e:
            rt.LoadedKModel(hip_ctx, data)
        return e.value.code

    assert code(b"KMDL" + good[4:]) == -rt.ERR_INVALID_MODEL_IDENTIFIER
    shipped_v5 = bytes.fromhex(GOLD["K14_kmodel_header_of_shipped_model"]["hex"])
    assert code(shipped_v5 + good[32:]) == -rt.ERR_INVALID_MODEL_VERSION
    assert code(good[:4] + struct.pack("<I", 6) + good[8:]) == -rt.ERR_INVALID_MODEL_VERSION
    other = km.KModel.parse(good)
    other.modules[0].kind = "stackvm"
    assert code(other.serialize()) == -rt.ERR_RUNTIME_NOT_FOUND      # no runtime for that module kind here
    import errno
    assert code(good[:20]) == -errno.EINVAL
    assert code(good[:len(good) // 2]) == -errno.EINVAL               # truncated inside the module
    no_entry = km.KModel.parse(good)
    no_entry.entry_module = km.MODEL_HAS_NO_ENTRY
    assert code(no_entry.serialize()) == -errno.EINVAL
    # an operator that reads a tensor nobody wrote, and weights pointing outside .rdata
    m = km.KModel.parse(good)
    tensors, ops, tin, tout = km.decode_hip_text(m.modules[0].section(".text").body)
    bad_ops = list(ops)
    bad_ops[1] = km.HipOp(ops[1].opcode, (3,), ops[1].output, ops[1].rdata0, ops[1].rdata1, ops[1].p, ops[1].f)
    for text in (km.encode_hip_text(tensors, bad_ops, tin, tout),
                 km.encode_hip_text(tensors, [ops[0], km.HipOp(ops[1].opcode, ops[1].inputs, ops[1].output, 1 << 40, ops[1].rdata1, ops[1].p, ops[1].f)] + list(ops[2:]), tin, tout)):
        mm = km.KModel.parse(good)
        mm.modules[0].sections[0].body = text
        mm.modules[0].functions[0].text_size = len(text)
        assert code(mm.serialize()) == -errno.EINVAL
    # extents whose product wraps 64 bits must not get past the size check
    huge = [km.HipTensor(t.dtype, (1 << 20, 1 << 20, 1 << 20, 1 << 20), t.zero_point, t.scale) if i == 2 else t for i, t in enumerate(tensors)]
    mm = km.KModel.parse(good)
    mm.modules[0].sections[0].body = km.encode_hip_text(huge, ops, tin, tout)
    assert code(mm.serialize()) == -errno.EINVAL
    unknown = [ops[0], km.HipOp(77, ops[1].inputs, ops[1].output)] + list(ops[2:])
    mm = km.KModel.parse(good)
    mm.modules[0].sections[0].body = km.encode_hip_text(tensors, unknown, tin, tout)
    assert code(mm.serialize()) == -rt.ERR_RUNTIME_NOT_FOUND
    rt.LoadedKModel(hip_ctx, good).destroy()                          # and the untouched file still loads


def test_stackvm_entry_that_extcalls_the_hip_function(hip_ctx):
    """The file form the compiler links -- module 0 `stackvm` whose main is LDARG 0; LDC_I4 function; LDC_I4 module;
    EXTCALL; RET, module 1 `hip` -- loads and gives the oracle's bytes like the single-module form; any other
    stackvm text is refused with runtime_not_found (there is no stackvm interpreter here)."""
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((8, 56, 56, 64), dtype=f32))
    x = rng.random((2, 56, 56, 64), dtype=f32)
    _, y_single, _ = run_and_check(hip_ctx, qg, x)
    _, y_two, _ = run_and_check(hip_ctx, qg, x, stackvm_main=True)
    assert np.array_equal(y_single.view(np.uint32), y_two.view(np.uint32))

    good = km.compile_quant_graph(qg, 2, stackvm_main=True)

    def code(model):
        with pytest.raises(rt.HipError) as e:
            rt.LoadedKModel(hip_ctx, model.serialize())
        return e.value.code

    def with_text(text):
        m = km.KModel.parse(good)
        m.modules[0].sections[0].body = text
        m.modules[0].functions[0].text_size = len(text)
        return m

    stub = km.stackvm_extcall_text(1, 0, 1)
    short_form = bytes([40]) + stub[3:]                                  # LDARG_0 instead of LDARG 0
    rt.LoadedKModel(hip_ctx, with_text(short_form).serialize()).destroy()
    assert code(with_text(stub[:-1])) == -rt.ERR_RUNTIME_NOT_FOUND        # no RET
    assert code(with_text(stub + bytes([93]))) == -rt.ERR_RUNTIME_NOT_FOUND
    assert code(with_text(bytes([1]) + stub)) == -rt.ERR_RUNTIME_NOT_FOUND   # LDNULL first: real stackvm code
    assert code(with_text(km.stackvm_extcall_text(1, 0, 0))) == -rt.ERR_RUNTIME_NOT_FOUND   # calls itself
    assert code(with_text(km.stackvm_extcall_text(1, 0, 7))) == -rt.ERR_RUNTIME_NOT_FOUND   # no such module
    import errno
    assert code(with_text(km.stackvm_extcall_text(1, 5, 1))) == -errno.EINVAL               # no such function
    assert code(with_text(km.stackvm_extcall_text(2, 0, 1))) == -rt.ERR_RUNTIME_NOT_FOUND   # main has one parameter


def test_sections_merged_into_rdata_are_resolved(hip_ctx):
    """A section flagged SECTION_MERGED_INTO_RDATA keeps its bytes inside .rdata (section.cpp:29-32): a hip module
    whose .text lives there loads to the same function."""
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(nb.conv_block(seed=1), rng.random((8, 56, 56, 64), dtype=f32))
    x = rng.random((1, 56, 56, 64), dtype=f32)
    plain = km.compile_quant_graph(qg, 1)
    want = rt.LoadedKModel(hip_ctx, plain).run(x)
    m = km.KModel.parse(plain)
    text, rdata = m.modules[0].section(".text").body, m.modules[0].section(".rdata").body
    pad = (-len(rdata)) % 64
    m.modules[0].sections[1].body = rdata + b"\0" * pad + text         # constants keep their offsets
    m.modules[0].sections[0].body = b""
    data = bytearray(m.serialize())
    pos = km.MODEL_HEADER.size + km.MODULE_HEADER.size + km.FUNCTION_HEADER.unpack_from(data, km.MODEL_HEADER.size + km.MODULE_HEADER.size)[-1]
    name, _flags, r0, size, _bs, _bz, mem = km.SECTION_HEADER.unpack_from(data, pos)
    assert name.rstrip(b"\0") == b".text"
    km.SECTION_HEADER.pack_into(data, pos, name, km.SECTION_MERGED_INTO_RDATA, r0, size, len(rdata) + pad, len(text), mem)
    got = rt.LoadedKModel(hip_ctx, bytes(data)).run(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_a_function_loads_from_its_text_and_rdata_spans(hip_ctx):
    """The entry point a hip runtime_function's initialize_core calls: the function's slice of the module's
    .text section plus the module's .rdata section give the same function as loading the whole file."""
    rng = np.random.default_rng(12)
    qg = nb.quantize_graph(nb.conv_block(seed=4), rng.random((8, 56, 56, 64), dtype=f32))
    x = rng.random((3, 56, 56, 64), dtype=f32)
    data = km.compile_quant_graph(qg, 3, stackvm_main=True)
    parsed = km.KModel.parse(data)
    hip = next(m for m in parsed.modules if m.kind == km.HIP_MODULE_KIND)
    secs = {s.name: s.body for s in hip.sections}
    fn = hip.functions[0]
    text = secs[".text"][fn.entrypoint:fn.entrypoint + fn.text_size]
    whole = rt.LoadedKModel(hip_ctx, data).run(x)
    part = rt.LoadedKModel(hip_ctx, text=text, rdata=secs[".rdata"])
    assert part.input_shape == x.shape
    assert np.array_equal(part.run(x).view(np.uint32), whole.view(np.uint32))
    with pytest.raises(rt.HipError) as e:                      # a constant that no longer fits the .rdata span
        rt.LoadedKModel(hip_ctx, text=text, rdata=secs[".rdata"][:64])
    assert e.value.code == -22
    with pytest.raises(rt.HipError) as e:
        rt.LoadedKModel(hip_ctx, text=text[:40], rdata=secs[".rdata"])
    assert e.value.code == -22


def test_a_matmul_function_with_f32_output_as_the_code_generator_writes_it(hip_ctx):
    """u8 [M, K] x u8 [K, N] -> f32 recorded as a 1x1 convolution over [M, 1, 1, K] with a float32 output tensor
    (the text the C# function builder emits for Dequantize -> MatMul without a Quantize consumer)."""
    from oracle import oracle as O
    rng = np.random.default_rng(21)
    M, K, N = 96, 160, 80
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    b = rng.integers(0, 256, (K, N), dtype=np.uint8)
    a_qp, b_qp = (7, 0.031), (131, 0.0123)
    rdata = km.RData()
    w_off = rdata.add(np.ascontiguousarray(b.T))            # OIHW = [N, K, 1, 1]
    tensors = [km.HipTensor("u8", (M, 1, 1, K), *a_qp), km.HipTensor("f32", (M, 1, 1, N))]
    inf = float(np.finfo(np.float32).max)
    ops = [km.HipOp(km.OP_CONV2D, (0,), 1, w_off, km.NO_RDATA, (N, K, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, b_qp[0]), (-inf, inf, b_qp[1]))]
    text = km.encode_hip_text(tensors, ops, 0, 1)
    model = rt.LoadedKModel(hip_ctx, text=text, rdata=bytes(rdata.buf))
    assert model.input_dtype == np.uint8 and model.output_dtype == np.float32
    got = model.run(a.reshape(M, 1, 1, K)).reshape(M, N)
    want = O.matmul_f32(O.dequantize(a, a_qp[1], a_qp[0]), O.dequantize(b, b_qp[1], b_qp[0]))
    # the device rounds the exact integer sum once; the float chain of the oracle rounds per term
    exact = ((a.astype(np.int64) - a_qp[0]) @ (b.astype(np.int64) - b_qp[0])).astype(np.float64) * (np.float32(a_qp[1]).astype(np.float64) * np.float32(b_qp[1]).astype(np.float64))
    assert np.abs(got - exact).max() <= np.abs(exact).max() * 2e-7 + 1e-6
    assert np.abs(got - want).max() <= np.abs(want).max() * 1e-4


def test_a_function_with_nchw_ends_as_the_code_generator_writes_it(hip_ctx):
    """What the C# function builder emits for an outlined region of a quantised network whose tensors the IR holds as
    NCHW: a layout step at the entry, every operator the lowering rules produce (conv, byte table, residual add,
    max pool, resize, concat, global mean), two outputs, and a layout step before each 4-D output."""
    from oracle import oracle as O
    rng = np.random.default_rng(33)
    N, C, H, W, OC = 2, 24, 20, 28, 24
    x = rng.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (OC, C, 3, 3), dtype=np.uint8)
    bias = rng.integers(-4000, 4000, OC, dtype=np.int32)
    qx, qw, qc, ql, qa, qp, qcat, qm = (120, 0.02), (128, 0.004), (110, 0.05), (8, 0.03), (100, 0.06), (90, 0.07), (95, 0.065), (97, 0.05)
    flt_max = float(np.finfo(np.float32).max)
    table = O.unary_lut(O.LUT_SWISH, *qc, *ql)

    rdata = km.RData()
    w_off, b_off, t_off = rdata.add(w), rdata.add(bias), rdata.add(table)
    T = km.HipTensor
    tensors = [
        T("u8", (N, H, W, C), *qx),             # 0 input as the caller hands it: N, C, H, W order
        T("u8", (N, H, W, C), *qx),             # 1 channels-last
        T("u8", (N, H, W, OC), *qc),            # 2 conv
        T("u8", (N, H, W, OC), *ql),            # 3 swish table
        T("u8", (N, H, W, OC), *qa),            # 4 add(3, 1)
        T("u8", (N, H // 2, W // 2, OC), *qp),  # 5 maxpool 2x2 / 2
        T("u8", (N, H, W, OC), *qp),            # 6 resize back to H x W
        T("u8", (N, H, W, 2 * OC), *qcat),      # 7 concat(6, 4)
        T("u8", (N, 1, 1, 2 * OC), *qm),        # 8 global mean: first output (H = W = 1 needs no layout step)
        T("u8", (N, H, W, 2 * OC), *qcat),      # 9 tensor 7 in N, C, H, W order: second output
    ]
    ops = [
        km.HipOp(km.OP_LAYOUT, (0,), 1, p=(0,)),
        km.HipOp(km.OP_CONV2D, (1,), 2, w_off, b_off, (OC, C, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, qw[0]), (-flt_max, flt_max, qw[1])),
        km.HipOp(km.OP_LUT, (2,), 3, t_off),
        km.HipOp(km.OP_ADD, (3, 1), 4, f=(0.0, 6.0)),
        km.HipOp(km.OP_MAXPOOL, (4,), 5, p=(2, 2, 0)),
        km.HipOp(km.OP_RESIZE_NEAREST, (5,), 6, p=(rt.RESIZE_ASYMMETRIC, rt.NEAREST_FLOOR)),
        km.HipOp(km.OP_CONCAT, (6, 4), 7),
        km.HipOp(km.OP_GLOBAL_AVGPOOL, (7,), 8),
        km.HipOp(km.OP_LAYOUT, (7,), 9, p=(1,)),
    ]
    for o in ops:  # the writer's field table describes every record used here
        pf, ff, nr = km.OP_FIELDS[km.OP_NAMES[o.opcode]]
        assert len(pf) == len(o.p) and len(ff) == len(o.f)
        assert nr == (o.rdata0 != km.NO_RDATA) + (o.rdata1 != km.NO_RDATA)
    text = km.encode_hip_text(tensors, ops, 0, 8, n_outputs=2)
    model = rt.LoadedKModel(hip_ctx, text=text, rdata=bytes(rdata.buf))
    assert len(model.outputs) == 2
    # the input buffer takes the caller's NCHW bytes as they are
    mean, cat = model.run(x.reshape(N, H, W, C))

    conv = O.qconv2d(x, w, bias, qx[0], qx[1], qw[0], qw[1], qc[0], qc[1], padding=((1, 1), (1, 1)))
    act = table[conv]
    add = O.qadd(act, x, ql[0], ql[1], qx[0], qx[1], qa[0], qa[1], fused_clamp=(0.0, 6.0))
    pool = O.qmaxpool(add, (2, 2), (2, 2), ((0, 0), (0, 0)), qa[0], qa[1], qp[0], qp[1])
    up = O.resize_nearest(pool, H, W, O.ASYMMETRIC, O.FLOOR)
    want_cat = O.qconcat([up, add], [qp, qa], qcat)
    want_mean = O.qglobal_avgpool(want_cat, qcat[0], qcat[1], qm[0], qm[1])
    assert np.array_equal(cat.reshape(N, 2 * OC, H, W), want_cat)
    assert np.array_equal(mean.reshape(N, 2 * OC), want_mean)
