"""kmodel v7 container and hip-module section format: byte layout against the reference's struct
definitions, round trips, and the compiler-side writer for quantised graphs (CPU only)."""
import json
import os
import struct

import numpy as np
import pytest

from nncase_amd import kmodel as km
from nncase_amd import netbuilder as nb

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def test_header_layout_matches_the_reference_structs():
    # model.h:38-74: model_header 8 x u32; module_header char[16] + 4 x u32 + u64;
    # function_header 2 x u32 + 3 x u64; section_header char[16] + 2 x u32 + 4 x u64
    assert (km.MODEL_HEADER.size, km.MODULE_HEADER.size, km.FUNCTION_HEADER.size, km.SECTION_HEADER.size) == (32, 40, 32, 56)
    shipped = bytes.fromhex(GOLD["K14_kmodel_header_of_shipped_model"]["hex"])
    assert len(shipped) == 32
    # the identifier this writer emits is byte for byte the one in the reference's own kmodel files
    blob = km.KModel([km.Module("hip", 1, [], [km.Section(".rdata", b"x")])]).serialize()
    assert blob[:4] == shipped[:4] == b"LDMK"
    assert struct.unpack_from("<I", blob, 4)[0] == 7 and struct.unpack_from("<I", shipped, 4)[0] == 5
    with pytest.raises(ValueError, match="version"):
        km.KModel.parse(shipped + b"\0" * 64)        # a version-5 file is refused (interpreter.cpp:99-102)
    with pytest.raises(ValueError, match="identifier"):
        km.KModel.parse(b"KMDL" + blob[4:])


def test_type_signatures():
    # type_serializer.cpp:24-72 / TypeSerializer.cs: 02 <typecode> 01 {01 <u32 dim>}* FF ; scalar: 02 <typecode> 00
    t = km.TensorType("f32", (1, 3, 224, 224))
    want = bytes([2, 0x0B, 1]) + b"".join(b"\x01" + struct.pack("<I", d) for d in (1, 3, 224, 224)) + b"\xff"
    assert km.encode_type(t) == want
    assert km.encode_type(km.TensorType("u8", None)) == bytes([2, 0x06, 0])
    assert km.encode_type(km.TensorType("f16", (None, 7))) == bytes([2, 0x0A, 1, 0, 1, 7, 0, 0, 0, 0xFF])
    tup = km.TupleType((t, km.TensorType("i32", None)))
    enc = km.encode_type(tup)
    assert enc[0] == 3 and enc[-1] == 0xFF
    for ty in (t, km.TensorType("u8", None), km.TensorType("f16", (None, 7)), tup):
        dec, pos = km.decode_type(km.encode_type(ty) + b"tail", 0)
        assert dec == ty and pos == len(km.encode_type(ty))


def test_container_round_trip_and_size_fields():
    rng = np.random.default_rng(5)
    def blob(n):
        return rng.integers(0, 256, n, dtype=np.uint8).tobytes()
    f0 = km.Function([km.TensorType("f32", (1, 3, 8, 8))], km.TensorType("f32", (1, 10)), 0, 17, [km.Section(".fsec", blob(5))])
    f1 = km.Function([], km.TupleType((km.TensorType("u8", (2,)),)), 17, 3)
    m0 = km.Module("stackvm", 1, [f0, f1], [km.Section(".text", blob(20)), km.Section(".rdata", blob(1000), alignment=128),
                                            km.Section(".custom_calls", struct.pack("<I16s", 1, b"hip"))])
    m1 = km.Module("hip", 1, [km.Function([km.TensorType("u8", (4,))], km.TensorType("u8", (4,)), 0, 9)],
                   [km.Section(".text", blob(9)), km.Section(".rdata", blob(77), flags=1, alignment=64, memory_size=4096)])
    data = km.KModel([m0, m1], entry_module=0, entry_function=1).serialize()
    assert len(data) % 8 == 0
    ident, ver, flags, align, nmod, em, ef, _ = km.MODEL_HEADER.unpack_from(data, 0)
    assert (ver, nmod, em, ef, align) == (7, 2, 0, 1, 128)        # alignment = lcm of the section alignments
    # module sizes chain to the end of the file; every size is a multiple of 8 and covers its header
    pos = 32
    for _ in range(2):
        size = km.MODULE_HEADER.unpack_from(data, pos)[-1]
        assert size % 8 == 0 and size >= 40
        pos += size
    assert pos == len(data)
    back = km.KModel.parse(data)
    assert [m.kind for m in back.modules] == ["stackvm", "hip"] and back.entry_function == 1
    for a, b in zip(back.modules, (m0, m1)):
        assert a.version == b.version and len(a.functions) == len(b.functions)
        for fa, fb in zip(a.functions, b.functions):
            assert (fa.parameter_types, fa.return_type, fa.entrypoint, fa.text_size) == (fb.parameter_types, fb.return_type, fb.entrypoint, fb.text_size)
            assert [(s.name, s.body) for s in fa.sections] == [(s.name, s.body) for s in fb.sections]
        for sa, sb in zip(a.sections, b.sections):
            assert (sa.name, sa.body, sa.flags) == (sb.name, sb.body, sb.flags)
            assert sa.body_start % sb.alignment == 0                # bodies start on their alignment
            assert sa.memory_size == (len(sb.body) if sb.memory_size is None else sb.memory_size)
    assert back.serialize() != b"" and km.KModel.parse(back.serialize()).modules[1].section(".rdata").body == m1.sections[1].body


def test_hip_module_of_a_quantised_graph():
    g = nb.conv_block(seed=1)
    rng = np.random.default_rng(1)
    qg = nb.quantize_graph(g, rng.random((4, 56, 56, 64), dtype=np.float32))
    data = km.compile_quant_graph(qg, batch=3)
    model = km.KModel.parse(data)
    assert model.entry_module == 0 and model.entry_function == 0 and model.modules[0].kind == "hip"
    fn = model.modules[0].functions[0]
    assert fn.parameter_types == [km.TensorType("f32", (3, 56, 56, 64))] and fn.return_type == km.TensorType("f32", (3, 56, 56, 64))
    text = model.modules[0].section(".text").body
    assert fn.entrypoint == 0 and fn.text_size == len(text)
    tensors, ops, tin, tout = km.decode_hip_text(text)
    assert [km.OP_NAMES[o.opcode] for o in ops] == ["quantize", "conv2d", "conv2d", "conv2d", "dequantize"]
    assert tin == 0 and tout == len(tensors) - 1 and tensors[0].dtype == "f32" and tensors[1].dtype == "u8"
    rdata = model.modules[0].section(".rdata").body
    convs = [n for n in qg.nodes if n.op == "conv"]
    for o, n in zip([o for o in ops if o.opcode == km.OP_CONV2D], convs):
        w = np.frombuffer(rdata, np.uint8, n.weights.size, o.rdata0).reshape(n.weights.shape)
        b = np.frombuffer(rdata, np.int32, n.bias.size, o.rdata1)
        assert np.array_equal(w, n.weights) and np.array_equal(b, n.bias)
        assert o.rdata0 % 64 == 0 and o.rdata1 % 64 == 0
        assert o.p[:5] == (*n.weights.shape, n.groups) and o.p[13] == n.w_qp[0]
        assert np.float32(o.f[2]) == np.float32(n.w_qp[1]) and np.float32(o.f[0]) == np.float32(n.clamp[0])
        assert (tensors[o.output].zero_point, np.float32(tensors[o.output].scale)) == (n.out_qp[0], np.float32(n.out_qp[1]))
    # a text survives its own round trip
    assert km.encode_hip_text(tensors, ops, tin, tout) == text
