"""kmodel v7 container (reader / writer) and the section format of the `hip` module.

Container layout, all little-endian (src/Native/include/nncase/runtime/model.h:38-74 ==
src/Nncase.CodeGen/CodeGen/KModelTypes.cs; writer order src/Nncase.CodeGen/CodeGen/LinkedModel.cs:28-172;
reader src/Native/src/runtime/interpreter.cpp:40-91, runtime_module.cpp:124-180):

    model_header   32 B  {u32 identifier 'KMDL' (bytes "LDMK"), version 7, flags, alignment, modules,
                          entry_module, entry_function, reserved0}
    per module:
      module_header 40 B {char kind[16]; u32 version, sections, functions, reserved0; u64 size}
      per function:
        function_header 32 B {u32 parameters, sections; u64 entrypoint, text_size, size}
        parameter type signatures, return type signature (type_serializer.cpp:24-97)
        function sections
      module sections
    section_header 56 B  {char name[16]; u32 flags, reserved0; u64 size, body_start, body_size, memory_size}

Every `size` includes its own header and the padding to 8 bytes that follows the body.  `body_start`
is the number of padding bytes between the end of the section header and the body (the writer stores
what AlignPosition returns, LinkedModel.cs:160 / CodeGenExtensions.cs:20-35; the reader adds it to the
position behind the header, src/Native/src/runtime/section.cpp:35-36,77-78).  A section whose flags
carry SECTION_MERGED_INTO_RDATA (1) has no body of its own: body_start is then an offset into the
body of the `.rdata` section of the same section list (section.cpp:29-32,71-76).

The `hip` module (kind "hip", version 1) holds one function whose `.text` is a flat operator list over
numbered NHWC tensors (HIPF format below) and a module section `.rdata` with the constants (u8 OIHW
weights, int32 biases, byte tables).  libnncase_hip.so loads such a module natively
(nncase_hip_kmodel_load); this file is the compiler-side writer and a generic reader.

HIPF (function text), 8-byte aligned records:
    header 32 B : "HIPF", u32 version=1, n_tensors, n_ops, input_tensor, output_tensor, n_outputs, reserved
                  (the outputs are tensors output_tensor .. output_tensor + n_outputs - 1; n_outputs 0 reads as 1)
    tensor 32 B : u32 dtype (typecode), rank, dims[4] (N, H, W, C), i32 zero_point, f32 scale
    op    144 B : u32 opcode, n_inputs; i32 inputs[8]; i32 output; u32 reserved;
                  u64 rdata0, rdata1 (offsets into .rdata, ~0 = none); i32 p[16]; f32 f[4]
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

MODEL_IDENTIFIER = 0x4B4D444C      # 'KMDL' as a C++ multi-character constant -> bytes 4C 44 4D 4B
MODEL_VERSION = 7
MODEL_HAS_NO_ENTRY = 0xFFFFFFFF
MIN_ALIGNMENT = 8
SECTION_MERGED_INTO_RDATA = 1      # model.h:76

MODEL_HEADER = struct.Struct("<8I")
MODULE_HEADER = struct.Struct("<16s4IQ")
FUNCTION_HEADER = struct.Struct("<2I3Q")
SECTION_HEADER = struct.Struct("<16s2I4Q")

# typecodes (src/Native/include/nncase/runtime/typecodes.def)
DT = {"bool": 0x00, "i8": 0x02, "i16": 0x03, "i32": 0x04, "i64": 0x05, "u8": 0x06, "u16": 0x07, "u32": 0x08, "u64": 0x09,
      "f16": 0x0A, "f32": 0x0B, "f64": 0x0C, "bf16": 0x0D}
DT_NAME = {v: k for k, v in DT.items()}
SIG_INVALID, SIG_ANY, SIG_TENSOR, SIG_TUPLE, SIG_CALLABLE, SIG_END = 0, 1, 2, 3, 4, 0xFF
DIM_UNKNOWN, DIM_FIXED = 0, 1


# ------------------------------------------------------------------------------------------------ type signatures
@dataclass(frozen=True)
class TensorType:
    dtype: str
    shape: Optional[Tuple[Optional[int], ...]]      # None = scalar; a None entry = unknown dimension


@dataclass(frozen=True)
class TupleType:
    fields: Tuple[object, ...]


def encode_type(t) -> bytes:
    if isinstance(t, TensorType):
        out = bytes([SIG_TENSOR, DT[t.dtype]])
        if t.shape is None:
            return out + b"\x00"
        out += b"\x01"
        for d in t.shape:
            out += bytes([DIM_UNKNOWN]) if d is None else bytes([DIM_FIXED]) + struct.pack("<I", d)
        return out + bytes([SIG_END])
    if isinstance(t, TupleType):
        return bytes([SIG_TUPLE]) + b"".join(encode_type(f) for f in t.fields) + bytes([SIG_END])
    raise TypeError(f"unsupported type {t!r}")


def decode_type(buf: bytes, pos: int):
    tok = buf[pos]
    pos += 1
    if tok == SIG_TENSOR:
        dtype = DT_NAME[buf[pos]]
        scalar = buf[pos + 1] == 0
        pos += 2
        if scalar:
            return TensorType(dtype, None), pos
        dims: List[Optional[int]] = []
        while buf[pos] != SIG_END:
            kind = buf[pos]
            pos += 1
            if kind == DIM_FIXED:
                dims.append(struct.unpack_from("<I", buf, pos)[0])
                pos += 4
            elif kind == DIM_UNKNOWN:
                dims.append(None)
            else:
                raise ValueError(f"invalid dim token {kind}")
        return TensorType(dtype, tuple(dims)), pos + 1
    if tok == SIG_TUPLE:
        fields = []
        while buf[pos] != SIG_END:
            f, pos = decode_type(buf, pos)
            fields.append(f)
        return TupleType(tuple(fields)), pos + 1
    raise ValueError(f"unsupported type signature token {tok}")


# ------------------------------------------------------------------------------------------------ container
@dataclass
class Section:
    name: str
    body: bytes
    flags: int = 0
    alignment: int = 8
    memory_size: Optional[int] = None
    body_start: int = 0          # header field, filled by the reader / writer: padding before the body
    body_pos: int = 0            # absolute position of the body in the file, filled by the reader / writer


@dataclass
class Function:
    parameter_types: List[object]
    return_type: object
    entrypoint: int = 0
    text_size: int = 0
    sections: List[Section] = field(default_factory=list)


@dataclass
class Module:
    kind: str
    version: int
    functions: List[Function] = field(default_factory=list)
    sections: List[Section] = field(default_factory=list)

    def section(self, name: str) -> Section:
        for s in self.sections:
            if s.name == name:
                return s
        raise KeyError(name)


@dataclass
class KModel:
    modules: List[Module]
    entry_module: int = MODEL_HAS_NO_ENTRY
    entry_function: int = MODEL_HAS_NO_ENTRY
    alignment: int = MIN_ALIGNMENT

    # ---- writer -------------------------------------------------------------------------------------
    def serialize(self) -> bytes:
        out = bytearray()

        def align(a: int):
            out.extend(b"\0" * ((-len(out)) % a))
            return len(out)

        def name16(s: str) -> bytes:
            b = s.encode("utf-8")
            if not 1 <= len(b) <= 16:
                raise ValueError(f"invalid name {s!r}")
            return b.ljust(16, b"\0")

        def write_section(s: Section):
            if s.flags & SECTION_MERGED_INTO_RDATA:
                raise ValueError("this writer keeps every section's body in the section itself")
            head = len(out)
            out.extend(b"\0" * SECTION_HEADER.size)
            s.body_pos = align(s.alignment)
            s.body_start = s.body_pos - (head + SECTION_HEADER.size)
            out.extend(s.body)
            end = align(MIN_ALIGNMENT)
            mem = len(s.body) if s.memory_size is None else s.memory_size
            SECTION_HEADER.pack_into(out, head, name16(s.name), s.flags, 0, end - head, s.body_start, len(s.body), mem)

        alignment = MIN_ALIGNMENT
        for m in self.modules:
            for s in m.sections:
                alignment = int(np.lcm(alignment, s.alignment))
        out.extend(MODEL_HEADER.pack(MODEL_IDENTIFIER, MODEL_VERSION, 0, alignment, len(self.modules), self.entry_module,
                                     self.entry_function, 0))
        for m in self.modules:
            mhead = len(out)
            out.extend(b"\0" * MODULE_HEADER.size)
            for f in m.functions:
                fhead = len(out)
                out.extend(b"\0" * FUNCTION_HEADER.size)
                for t in f.parameter_types:
                    out.extend(encode_type(t))
                out.extend(encode_type(f.return_type))
                for s in f.sections:
                    write_section(s)
                end = align(MIN_ALIGNMENT)
                FUNCTION_HEADER.pack_into(out, fhead, len(f.parameter_types), len(f.sections), f.entrypoint, f.text_size, end - fhead)
            for s in m.sections:
                write_section(s)
            end = align(MIN_ALIGNMENT)
            MODULE_HEADER.pack_into(out, mhead, name16(m.kind), m.version, len(m.sections), len(m.functions), 0, end - mhead)
        return bytes(out)

    # ---- reader -------------------------------------------------------------------------------------
    @staticmethod
    def parse(buf: bytes) -> "KModel":
        ident, version, _flags, alignment, n_modules, entry_module, entry_function, _ = MODEL_HEADER.unpack_from(buf, 0)
        if ident != MODEL_IDENTIFIER:
            raise ValueError("invalid model identifier")       # nncase_errc::invalid_model_indentifier
        if version != MODEL_VERSION:
            raise ValueError(f"invalid model version {version}")  # nncase_errc::invalid_model_version

        def read_sections(pos: int, count: int):
            """`count` section records from `pos`: bodies located like runtime::find_section (section.cpp:58-91)."""
            heads = []
            for _ in range(count):
                name, flags, _r, size, body_start, body_size, memory_size = SECTION_HEADER.unpack_from(buf, pos)
                if size < SECTION_HEADER.size or pos + size > len(buf):
                    raise ValueError("bad section size")
                heads.append((name.rstrip(b"\0").decode(), flags, pos, body_start, body_size, memory_size))
                pos += size
            rdata_pos = next((hp + SECTION_HEADER.size + bs for n, f, hp, bs, _z, _m in heads
                              if n == ".rdata" and not f & SECTION_MERGED_INTO_RDATA), None)
            out = []
            for name, flags, hp, body_start, body_size, memory_size in heads:
                if flags & SECTION_MERGED_INTO_RDATA:
                    if rdata_pos is None:
                        raise ValueError(f"section {name} is merged into a .rdata section that does not exist")
                    body_pos = rdata_pos + body_start
                else:
                    body_pos = hp + SECTION_HEADER.size + body_start
                if body_pos + body_size > len(buf):
                    raise ValueError(f"section {name} body outside the file")
                out.append(Section(name, bytes(buf[body_pos:body_pos + body_size]), flags, 8, memory_size, body_start, body_pos))
            return out, pos

        modules = []
        pos = MODEL_HEADER.size
        for _ in range(n_modules):
            kind, mver, n_sections, n_functions, _r, msize = MODULE_HEADER.unpack_from(buf, pos)
            m = Module(kind.rstrip(b"\0").decode(), mver)
            p = pos + MODULE_HEADER.size
            for _f in range(n_functions):
                n_params, n_fsec, entrypoint, text_size, fsize = FUNCTION_HEADER.unpack_from(buf, p)
                q = p + FUNCTION_HEADER.size
                params = []
                for _p in range(n_params):
                    t, q = decode_type(buf, q)
                    params.append(t)
                ret, q = decode_type(buf, q)
                fn = Function(params, ret, entrypoint, text_size)
                fn.sections, q = read_sections(q, n_fsec)
                m.functions.append(fn)
                p += fsize
            m.sections, p = read_sections(p, n_sections)
            modules.append(m)
            pos += msize
        return KModel(modules, entry_module, entry_function, alignment)


# ------------------------------------------------------------------------------------------------ hip module
HIP_MODULE_KIND = "hip"
HIP_MODULE_VERSION = 1
HIPF_MAGIC = b"HIPF"
HIPF_VERSION = 1
HIPF_HEADER = struct.Struct("<4s7I")
HIPF_TENSOR = struct.Struct("<6Iif")
HIPF_OP = struct.Struct("<2I8iiI2Q16i4f")
NO_RDATA = 0xFFFFFFFFFFFFFFFF
(OP_QUANTIZE, OP_DEQUANTIZE, OP_CONV2D, OP_ADD, OP_GLOBAL_AVGPOOL, OP_LUT, OP_CONCAT, OP_RESIZE_NEAREST, OP_MAXPOOL,
 OP_PAD_CHANNELS, OP_RESHAPE, OP_LAYOUT) = range(12)
OP_NAMES = ["quantize", "dequantize", "conv2d", "add", "global_avgpool", "lut", "concat", "resize_nearest", "maxpool",
            "pad_channels", "reshape", "layout"]
# What each operator record holds beside its tensors: names of p[0..], names of f[0..], number of .rdata offsets.
# (The loader, nncase_hip_kmodel_load_function, and the compiler-side writer follow this table field by field.)
OP_FIELDS = {
    "quantize": ((), (), 0),
    "dequantize": ((), (), 0),
    "conv2d": (("out_channels", "group_in_channels", "kernel_h", "kernel_w", "groups", "stride_h", "stride_w", "dilation_h",
                "dilation_w", "pad_h_before", "pad_h_after", "pad_w_before", "pad_w_after", "weights_zero_point"),
               ("clamp_min", "clamp_max", "weights_scale"), 2),
    "add": ((), ("clamp_min", "clamp_max"), 0),
    "global_avgpool": ((), (), 0),
    "lut": ((), (), 1),
    "concat": ((), (), 0),
    "resize_nearest": (("transformation_mode", "nearest_mode"), (), 0),
    "maxpool": (("kernel", "stride", "padding"), (), 0),
    "pad_channels": ((), (), 0),
    "reshape": ((), (), 0),
    "layout": (("to_nchw",), (), 0),     # the tensor on the NCHW side still records its extents as N, H, W, C
}
assert list(OP_FIELDS) == OP_NAMES
assert HIPF_HEADER.size == 32 and HIPF_TENSOR.size == 32 and HIPF_OP.size == 144


@dataclass
class HipTensor:
    dtype: str
    dims: Tuple[int, int, int, int]     # N, H, W, C
    zero_point: int = 0
    scale: float = 1.0


@dataclass
class HipOp:
    opcode: int
    inputs: Tuple[int, ...]
    output: int
    rdata0: int = NO_RDATA
    rdata1: int = NO_RDATA
    p: Tuple[int, ...] = ()
    f: Tuple[float, ...] = ()


class RData:
    """Constant pool: 64-byte aligned blobs."""

    def __init__(self):
        self.buf = bytearray()

    def add(self, arr: np.ndarray) -> int:
        self.buf.extend(b"\0" * ((-len(self.buf)) % 64))
        off = len(self.buf)
        self.buf.extend(np.ascontiguousarray(arr).tobytes())
        return off


def encode_hip_text(tensors: Sequence[HipTensor], ops: Sequence[HipOp], input_tensor: int, output_tensor: int,
                    n_outputs: int = 1) -> bytes:
    out = bytearray(HIPF_HEADER.pack(HIPF_MAGIC, HIPF_VERSION, len(tensors), len(ops), input_tensor, output_tensor,
                                     0 if n_outputs == 1 else n_outputs, 0))
    for t in tensors:
        out.extend(HIPF_TENSOR.pack(DT[t.dtype], 4, *t.dims, int(t.zero_point), float(np.float32(t.scale))))
    for o in ops:
        ins = tuple(o.inputs) + (-1,) * (8 - len(o.inputs))
        p = tuple(int(v) for v in o.p) + (0,) * (16 - len(o.p))
        f = tuple(float(np.float32(v)) for v in o.f) + (0.0,) * (4 - len(o.f))
        out.extend(HIPF_OP.pack(o.opcode, len(o.inputs), *ins, o.output, 0, o.rdata0, o.rdata1, *p, *f))
    return bytes(out)


def decode_hip_text(text: bytes):
    magic, version, n_tensors, n_ops, input_tensor, output_tensor, _n_outputs, _ = HIPF_HEADER.unpack_from(text, 0)
    if magic != HIPF_MAGIC or version != HIPF_VERSION:
        raise ValueError("not a hip function text")
    pos = HIPF_HEADER.size
    tensors, ops = [], []
    for _ in range(n_tensors):
        dt, _rank, n, h, w, c, zp, sc = HIPF_TENSOR.unpack_from(text, pos)
        tensors.append(HipTensor(DT_NAME[dt], (n, h, w, c), zp, sc))
        pos += HIPF_TENSOR.size
    for _ in range(n_ops):
        v = HIPF_OP.unpack_from(text, pos)
        opcode, n_in = v[0], v[1]
        ops.append(HipOp(opcode, tuple(v[2:2 + n_in]), v[10], v[12], v[13], tuple(v[14:30]), tuple(v[30:34])))
        pos += HIPF_OP.size
    return tensors, ops, input_tensor, output_tensor


# ------------------------------------------------------------------------------------------------ stackvm entry stub
STACKVM_MODULE_KIND = "stackvm"
STACKVM_MODULE_VERSION = 1          # modules/Nncase.Modules.StackVM/Runtime/StackVM/StackVMRTModule.cs
# src/Native/include/nncase/runtime/stackvm/opcode.h:26-127
OPC_LDC_I4, OPC_LDARG, OPC_RET, OPC_EXTCALL = 2, 39, 93, 96


def stackvm_extcall_text(n_args: int, function_id: int, module_id: int, is_prim_func: bool = False) -> bytes:
    """The stackvm text the compiler emits for `main(args) = callee(args)` with the callee in another module
    (modules/Nncase.Modules.StackVM/CodeGen/StackVM/CodegenVisitor.cs:281-315: arguments visited in reverse,
    then LdFunctionId :470-476 = LDC_I4 function id, LDC_I4 module id, then EXTCALL, and RET :244).
    Encodings (op_reader.h): opcode u8; LDARG u16 index; LDC_I4 i32; EXTCALL u16 args + u8 is_prim_func."""
    out = bytearray()
    for i in reversed(range(n_args)):
        out += struct.pack("<BH", OPC_LDARG, i)
    out += struct.pack("<Bi", OPC_LDC_I4, function_id)
    out += struct.pack("<Bi", OPC_LDC_I4, module_id)
    out += struct.pack("<BHB", OPC_EXTCALL, n_args, 1 if is_prim_func else 0)
    out += struct.pack("<B", OPC_RET)
    return bytes(out)


def with_stackvm_main(callee: Module, function_index: int = 0) -> "KModel":
    """A two-module kmodel as the compiler links it: module 0 = `stackvm` whose only function calls function
    `function_index` of module 1 = `callee` through EXTCALL; the model's entry is the stackvm function.
    `.custom_calls` holds a zero count (u32 count + count x char[16], StackVMLinkableModule.cs ctor; reader
    src/Native/src/runtime/stackvm/runtime_module.cpp:35-54)."""
    f = callee.functions[function_index]
    text = stackvm_extcall_text(len(f.parameter_types), function_index, 1)
    main = Function(list(f.parameter_types), f.return_type, 0, len(text))
    vm = Module(STACKVM_MODULE_KIND, STACKVM_MODULE_VERSION, [main],
                [Section(".text", text), Section(".rdata", b""), Section(".custom_calls", struct.pack("<I", 0))])
    return KModel([vm, callee], entry_module=0, entry_function=0)


def compile_quant_graph(qg, batch: int, stackvm_main: bool = False) -> bytes:
    """Emits a kmodel for a netbuilder.QuantGraph at a fixed batch: f32 NHWC input -> quantize -> the graph's
    u8 operators -> dequantize -> f32 output, as one function of a module of kind "hip".  With stackvm_main the
    file has the shape the compiler links: its entry is a `stackvm` function that EXTCALLs the hip function."""
    rdata = RData()
    tensors: List[HipTensor] = []
    ops: List[HipOp] = []
    c0, h0, w0 = qg.nodes[0].out_shape
    tensors.append(HipTensor("f32", (batch, h0, w0, c0)))
    node_tensor: Dict[int, int] = {}
    for i, n in enumerate(qg.nodes):
        c, h, w = n.out_shape
        tensors.append(HipTensor("u8", (batch, h, w, c), int(n.out_qp[0]), float(n.out_qp[1])))
        tid = len(tensors) - 1
        node_tensor[i] = tid
        ins = tuple(node_tensor[j] for j in n.inputs)
        if n.op == "input":
            ops.append(HipOp(OP_QUANTIZE, (0,), tid))
        elif n.op == "conv":
            oc, gic, kh, kw = n.weights.shape
            w_off = rdata.add(n.weights.astype(np.uint8))
            b_off = NO_RDATA if n.bias is None else rdata.add(n.bias.astype(np.int32))
            (ph0, ph1), (pw0, pw1) = n.padding
            ops.append(HipOp(OP_CONV2D, ins, tid, w_off, b_off,
                             (oc, gic, kh, kw, n.groups, n.stride[0], n.stride[1], 1, 1, ph0, ph1, pw0, pw1, int(n.w_qp[0])),
                             (n.clamp[0], n.clamp[1], float(n.w_qp[1]))))
        elif n.op == "add":
            clamp = getattr(n, "clamp", None) or (-3.4028234663852886e38, 3.4028234663852886e38)
            ops.append(HipOp(OP_ADD, ins, tid, f=(clamp[0], clamp[1])))
        elif n.op == "gap":
            ops.append(HipOp(OP_GLOBAL_AVGPOOL, ins, tid))
        elif n.op == "lut":
            ops.append(HipOp(OP_LUT, ins, tid, rdata.add(np.asarray(n.lut, np.uint8))))
        elif n.op == "concat":
            ops.append(HipOp(OP_CONCAT, ins, tid))
        elif n.op == "resize":
            ops.append(HipOp(OP_RESIZE_NEAREST, ins, tid, p=(n.resize_modes[0], n.resize_modes[1])))
        elif n.op == "maxpool":
            ops.append(HipOp(OP_MAXPOOL, ins, tid, p=(n.pool[0], n.pool[1], n.pool[2])))
        elif n.op == "padc":
            ops.append(HipOp(OP_PAD_CHANNELS, ins, tid))
        elif n.op == "s2d":        # channel padding to 4 and 2 x 2 pixel blocks to 16-channel pixels (extents say which)
            ops.append(HipOp(OP_PAD_CHANNELS, ins, tid))
        elif n.op == "fold2":      # the same NHWC bytes with other extents: the tensor shares its input's buffer
            ops.append(HipOp(OP_RESHAPE, ins, tid))
        else:
            raise ValueError(f"cannot serialise operator {n.op!r}")
    first_out = len(tensors)
    out_types = []
    for j in qg.output_nodes:
        c, h, w = qg.nodes[j].out_shape
        tensors.append(HipTensor("f32", (batch, h, w, c)))
        ops.append(HipOp(OP_DEQUANTIZE, (node_tensor[j],), len(tensors) - 1))
        out_types.append(TensorType("f32", tensors[-1].dims))
    text = encode_hip_text(tensors, ops, 0, first_out, len(out_types))
    ret = out_types[0] if len(out_types) == 1 else TupleType(tuple(out_types))
    fn = Function([TensorType("f32", tensors[0].dims)], ret, 0, len(text))
    mod = Module(HIP_MODULE_KIND, HIP_MODULE_VERSION, [fn],
                 [Section(".text", text), Section(".rdata", bytes(rdata.buf), alignment=64)])
    if stackvm_main:
        return with_stackvm_main(mod).serialize()
    return KModel([mod], entry_module=0, entry_function=0).serialize()
