"""The C-ABI library loads on a machine without a GPU and exports every symbol that
include/nncase_hip.h declares; argument checks that need no device return the documented
error codes.  No compute call is made here."""
import ctypes as C
import errno
import os
import re

import pytest

from nncase_amd import runtime as rt

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "nncase_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"NNCASE_HIP_API\s+[\w\s\*]+?\b(nncase_hip_\w+)\s*\(", text)))


def test_header_and_binding_table_agree():
    assert declared_symbols() == sorted(rt.SYMBOLS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(rt.LIB_PATH), "build with `python -m nncase_amd.build`"
    lib = C.CDLL(rt.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in nncase_hip.h but not exported"


def test_null_handles_are_einval_without_a_device():
    lib = rt.load_library()
    assert lib.nncase_hip_version() >= 1
    assert lib.nncase_hip_ctx_create(0, None) == -errno.EINVAL
    assert lib.nncase_hip_ctx_destroy(None) == -errno.EINVAL
    assert lib.nncase_hip_stream_sync(None) == -errno.EINVAL
    assert lib.nncase_hip_malloc(None, 16, None) == -errno.EINVAL
    assert lib.nncase_hip_quantize(None, None, rt.DT_F32, None, rt.DT_U8, 4, rt.qp(0, 1.0)) == -errno.EINVAL
    assert lib.nncase_hip_qconv2d(None, None, None, None, None) == -errno.EINVAL
    assert lib.nncase_hip_paged_attention_decode(None, None, None, None, None, None, None, None) == -errno.EINVAL
    assert lib.nncase_hip_last_error_string(None) == b""


def test_struct_layouts_match_the_header():
    # fixed-layout PODs: sizes the C side was compiled with
    assert C.sizeof(rt.QuantParam) == 8
    assert C.sizeof(rt.Conv2dDesc) == 5 * 4 + 8 + 4 + 8  # 4 bytes of padding before the int64
    assert C.sizeof(rt.Conv2dArgs) == 11 * 4 + 8 + 8 + 3 * 4 + 8 + 8 + 8 + 2 * 4 + 2 * 4 + 2 * 4
    assert C.sizeof(rt.MatmulArgs) == 4 + 8 + 8 + 3 * 4
    assert C.sizeof(rt.QBlockDesc) == 3 * 4 + 3 * 8 and C.sizeof(rt.QBlockArgs) == 8 * 4 + 4 * 8 + 6 * 4 + 4 + 8 + 2 * 4
    assert C.sizeof(rt.PagedAttnArgs) == 10 * 4


# ---- the three descriptions of every POD agree field by field: the C header, the ctypes binding, the C# binding ----
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CS_NATIVE = os.path.join(ROOT, "modules", "Nncase.Modules.Hip", "Interop", "NativeMethods.cs")
CS_BUILDER = os.path.join(ROOT, "modules", "Nncase.Modules.Hip", "CodeGen", "Hip", "HipModuleBuilder.cs")
KIND = {"int32_t": "i32", "int64_t": "i64", "float": "f32", "nncase_hip_quant_param_t": "qp",
        "int": "i32", "long": "i64", "IntPtr": "ptr", "HipQuantParam": "qp"}
SIZE_ALIGN = {"i32": (4, 4), "f32": (4, 4), "i64": (8, 8), "ptr": (8, 8), "qp": (8, 4)}
PODS = {  # header typedef -> (C# struct, ctypes class)
    "nncase_hip_quant_param_t": ("HipQuantParam", rt.QuantParam),
    "nncase_hip_conv2d_desc_t": ("HipConv2DDesc", rt.Conv2dDesc),
    "nncase_hip_conv2d_args_t": ("HipConv2DArgs", rt.Conv2dArgs),
    "nncase_hip_qblock_desc_t": ("HipQBlockDesc", rt.QBlockDesc),
    "nncase_hip_qblock_args_t": ("HipQBlockArgs", rt.QBlockArgs),
    "nncase_hip_matmul_args_t": ("HipMatMulArgs", rt.MatmulArgs),
    "nncase_hip_paged_attn_args_t": ("HipPagedAttnArgs", rt.PagedAttnArgs),
}


def layout(kinds):
    """Offsets and size of a C struct with natural alignment (what LayoutKind.Sequential also produces)."""
    off, offsets, worst = 0, [], 1
    for k in kinds:
        size, align = SIZE_ALIGN[k]
        off = (off + align - 1) // align * align
        offsets.append(off)
        off += size
        worst = max(worst, align)
    return offsets, (off + worst - 1) // worst * worst


def header_structs():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for m in re.finditer(r"typedef struct \w+ \{(.*?)\} (\w+);", text, re.S):
        fields = []
        for decl in m.group(1).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            if "*" in decl:
                fields.append(("ptr", decl.split("*")[-1].strip()))
                continue
            ctype, names = decl.split(" ", 1)
            fields += [(KIND[ctype], n.strip()) for n in names.split(",")]
        out[m.group(2)] = fields
    return out


def csharp_structs():
    text = open(CS_NATIVE).read()
    out = {}
    for m in re.finditer(r"\[StructLayout\(LayoutKind\.Sequential\)\]\s*public struct (\w+)\s*\{(.*?)\n\}", text, re.S):
        out[m.group(1)] = [(KIND[t], n) for t, n in re.findall(r"^\s*public (\w+) (\w+);", m.group(2), re.M)]
    return out


def test_header_ctypes_and_csharp_pods_agree():
    hs, cs = header_structs(), csharp_structs()
    assert set(hs) == set(PODS), "a POD of the header has no C# / ctypes counterpart listed here"
    for hname, (csname, ctype) in PODS.items():
        hk = [k for k, _ in hs[hname]]
        assert [k for k, _ in cs[csname]] == hk, f"{csname} field types / order differ from {hname}"
        # C# PascalCase names are the header's snake_case names
        assert [n.lower() for _, n in cs[csname]] == [n.replace("_", "") for _, n in hs[hname]], csname
        offsets, size = layout(hk)
        assert C.sizeof(ctype) == size, hname
        assert [getattr(ctype, f[0]).offset for f in ctype._fields_] == offsets, hname
        assert [f[0] for f in ctype._fields_] == [n for _, n in hs[hname]], hname
    assert layout([k for k, _ in hs["nncase_hip_conv2d_args_t"]])[1] == 120


def test_csharp_imports_name_exported_symbols_with_the_right_arity():
    header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    arity = {}
    for m in re.finditer(r"NNCASE_HIP_API\s+[\w\s\*]+?\b(nncase_hip_\w+)\s*\((.*?)\)\s*;", header, re.S):
        args = m.group(2).strip()
        arity[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    cs = open(CS_NATIVE).read()
    imports = re.findall(r"public static extern \w+ (nncase_hip_\w+)\((.*?)\);", cs, re.S)
    assert len(imports) >= 20
    for name, args in imports:
        assert name in arity, f"{name} is imported by the C# binding but not declared in the header"
        assert (args.count(",") + 1 if args.strip() else 0) == arity[name], name


def test_csharp_function_text_constants_match_the_writer():
    from nncase_amd import kmodel as km
    cs = open(CS_BUILDER).read()
    const = {k: int(v) for k, v in re.findall(r"public const (?:int|uint) (\w+) = (\d+);", cs)}
    assert const["HeaderBytes"] == km.HIPF_HEADER.size and const["TensorBytes"] == km.HIPF_TENSOR.size
    assert const["OpBytes"] == km.HIPF_OP.size and const["TextVersion"] == km.HIPF_VERSION
    assert const["RdataAlignment"] == 64
    body = re.search(r"internal enum HipOpcode : uint\s*\{(.*?)\}", cs, re.S).group(1)
    opcodes = {n.lower(): int(v) for n, v in re.findall(r"(\w+) = (\d+),", body)}
    assert opcodes == {n.replace("_", ""): i for i, n in enumerate(km.OP_NAMES)}
    assert '"HIPF"' in cs and km.HIPF_MAGIC == b"HIPF"


CS_MODULE = os.path.join(ROOT, "modules", "Nncase.Modules.Hip")


def cs(*parts):
    return open(os.path.join(CS_MODULE, *parts)).read()


def csharp_op_layouts():
    """HipOpLayouts.Fields of the function builder, as {opcode name: (p names, f names, rdata count)}."""
    body = re.search(r"class HipOpLayouts\s*\{(.*?)\n\}", cs("CodeGen", "Hip", "HipModuleBuilder.cs"), re.S).group(1)
    out = {}
    for entry in body.split("[HipOpcode.")[1:]:
        name, value = entry.split("]", 1)
        value = value[:value.rindex("),")]
        lists = [tuple(re.findall(r'"(\w+)"', m.group(1) or ""))
                 for m in re.finditer(r"new string\[0\]|new\[\] \{(.*?)\}", value, re.S)]
        assert len(lists) == 2, name
        out[name] = (lists[0], lists[1], int(re.search(r"(\d+)\s*$", value).group(1)))
    return out


def test_csharp_operator_records_follow_the_writers_field_table():
    from nncase_amd import kmodel as km
    layouts = csharp_op_layouts()
    assert {n.lower(): v for n, v in layouts.items()} == {n.replace("_", ""): v for n, v in km.OP_FIELDS.items()}


def test_loader_reads_exactly_the_fields_the_table_names():
    """Every `case kOpX:` of the loader indexes p[] and f[] of its record below the table's lengths, and uses them all."""
    from nncase_amd import kmodel as km
    text = open(os.path.join(ROOT, "nncase_amd", "csrc", "kmodel.hip")).read()
    enum = re.search(r"enum \{ (kOpQuantize.*?) \};", text, re.S).group(1)
    names = [n.strip() for n in enum.replace("\n", " ").split(",")]
    assert [n[3:].lower() for n in names] == [n.replace("_", "") for n in km.OP_NAMES]
    switch = text[text.index("switch (o.opcode) {"):]
    blocks = re.split(r"\n        case (kOp\w+):", switch[:switch.index("\n        default:")])
    seen = {}
    for label, block in zip(blocks[1::2], blocks[2::2]):
        if label == "kOpConv2d":     # its record is read by the helper that a pair's other convolutions go through as well
            assert "prepare_conv(k," in block
            block = text[text.index("auto prepare_conv = "):text.index("    for (uint32_t k = 0; k < th.n_ops; k++) {", text.index("auto prepare_conv = "))]
        seen[label] = ({int(i) for i in re.findall(r"\bo\.p\[(\d+)\]", block)}, {int(i) for i in re.findall(r"\bo\.f\[(\d+)\]", block)},
                       len(set(re.findall(r"\bo\.rdata(\d)", block))))
    assert set(seen) == set(names)
    for label, name in zip(names, km.OP_NAMES):
        p, f, r = seen[label]
        pn, fn, rn = km.OP_FIELDS[name]
        assert p == set(range(len(pn))) and f == set(range(len(fn))) and r == rn, (name, p, f, r)


def test_every_opcode_and_operator_of_the_csharp_module_is_wired_through():
    """Each opcode has an emitter; each hip operator has a lowering rule that the target registers, a case in the
    function builder and an evaluator that the plugin registers."""
    from nncase_amd import kmodel as km
    builder = cs("CodeGen", "Hip", "HipModuleBuilder.cs")
    emitted = set(re.findall(r"AddOp\(\s*HipOpcode\.(\w+)", builder))
    assert {n.lower() for n in emitted} == {n.replace("_", "") for n in km.OP_NAMES}
    ops = re.findall(r"public sealed partial class (Hip\w+) : Op, IHipOp", cs("IR", "Hip", "HipOps.cs"))
    assert len(ops) == 11
    rules = "".join(cs("Passes", "Rules", "Hip", f) for f in os.listdir(os.path.join(CS_MODULE, "Passes", "Rules", "Hip")))
    target, plugin = cs("Targets", "HipTarget.cs"), cs("HipModule.cs")
    evaluators = cs("Evaluator", "Hip", "HipEvaluators.cs") + cs("Evaluator", "Hip", "HipRaisedEvaluators.cs")
    for op in ops:
        assert re.search(r"case %s\b" % op, builder), f"{op}: no case in the function builder"
        made_by = [r for r, body in re.findall(r"public sealed partial class (\w+) : IRewriteRule(.*?)(?=\n\[RuleGenerator\]|\ninternal static class|\Z)", rules, re.S)
                   if re.search(r"new %s\b" % op, body) or (op == "HipQConcat" and "HipConcat.Build" in body)]
        assert made_by and all(f"p.Add<{r}>()" in target for r in made_by), f"{op}: rules {made_by} not registered"
        ev = re.search(r"class (\w+) : (?:HipRaisedEvaluator<%s>|IEvaluator<%s>)" % (op, op), evaluators)
        assert ev and f"RegisterManyInterface<{ev.group(1)}>" in plugin, f"{op}: evaluator missing or not registered"
    # the outlining pass builds what the unmodified stackvm code generator accepts: a wrapper over a prim function
    outline = cs("Passes", "OutlineHipFunctionsPass.cs")
    assert "new PrimFunctionWrapper(" in outline and "new PrimFunction(" in outline and "new Fusion(" not in outline
    assert "(TIR.PrimFunction)callable" in builder


def test_errno_statuses_stay_clear_of_the_nncase_errc_block():
    """A status in [-7, -1] must always be an nncase_errc: the runtime-module shim maps statuses back by range."""
    src = os.path.join(ROOT, "nncase_amd", "csrc")
    used = set()
    for f in os.listdir(src):
        used |= set(re.findall(r"-(E[A-Z0-9]+)\b", open(os.path.join(src, f)).read()))
    used -= {"ERR"}
    assert used and all(getattr(errno, name) > 7 for name in used), sorted(used)


# ---- the runtime-module shim (C++ against the reference's headers, not compilable here) is checked as text ----
SHIM_DIR = os.path.join(ROOT, "modules", "hip", "src", "runtime")
REF_ERRC_BLOCK = {  # src/Native/include/nncase/runtime/error.h:21-37, the values a hip module can report
    "INVALID_MODEL_IDENTIFIER": 0x01, "INVALID_MODEL_VERSION": 0x03, "RUNTIME_NOT_FOUND": 0x04,
    "DATATYPE_MISMATCH": 0x05, "SHAPE_MISMATCH": 0x06, "INVALID_MEMORY_LOCATION": 0x07,
}


def shim_sources():
    return {f: open(os.path.join(SHIM_DIR, f)).read() for f in sorted(os.listdir(SHIM_DIR))}


def shim_status_map():
    """to_error_code of the shim, rebuilt from its text: the two thresholds and the order of the tests."""
    text = shim_sources()["runtime_module.cpp"]
    last = int(re.search(r"NNCASE_ERRC_LAST\s*=\s*(0x[0-9a-fA-F]+|\d+)\s*;", text).group(1), 0)
    base = int(re.search(r"HIP_STATUS_BASE\s*=\s*(0x[0-9a-fA-F]+|\d+)\s*;", text).group(1), 0)
    body = text[text.index("to_error_code(int rc) noexcept {"):]
    body = body[:body.index("\n}\n")]
    tests_in_order = re.findall(r"if \(rc (>=|<=) -(\w+)\)\s*return ([^;]+);", body)
    assert [(op, name) for op, name, _ in tests_in_order] == [(">=", "NNCASE_ERRC_LAST"), ("<=", "HIP_STATUS_BASE")], tests_in_order
    assert "nncase_errc" in tests_in_order[0][2] and "io_error" in tests_in_order[1][2]
    assert re.search(r"return std::make_error_code\(static_cast<std::errc>\(-rc\)\);\s*$", body), "the rest is -errno"

    def classify(rc):
        if rc >= -last:
            return ("nncase_errc", -rc)
        if rc <= -base:
            return ("io_error", None)
        return ("errno", -rc)
    return classify, last, base


def test_shim_maps_every_library_status_to_the_right_category():
    header = open(HEADER).read()
    enum = {n: int(v, 0) for n, v in re.findall(r"NNCASE_HIP_ERR_(\w+) = (0x[0-9a-fA-F]+)", header)}
    hip_base = enum.pop("HIP_BASE")
    assert enum == REF_ERRC_BLOCK, "the header's first error block is nncase_errc's"
    classify, last, base = shim_status_map()
    assert last == max(enum.values()) and base == hip_base
    for name, value in enum.items():
        assert classify(-value) == ("nncase_errc", value), name
    # every errno the library returns keeps its meaning, whichever side of 0x100 it lies on
    src = os.path.join(ROOT, "nncase_amd", "csrc")
    used = set()
    for f in os.listdir(src):
        used |= set(re.findall(r"-(E[A-Z0-9]+)\b", open(os.path.join(src, f)).read()))
    used -= {"ERR"}
    for name in used:
        assert classify(-getattr(errno, name)) == ("errno", getattr(errno, name)), name
    # a failed HIP runtime call: -(0x1000 + hipError_t), hipError_t in [1, 1054] on this runtime
    for hip_error in (1, 2, 98, 700, 719, 999, 1054):
        assert classify(-(hip_base + hip_error)) == ("io_error", None)
    # the library itself keeps the block clear (what makes the first test of the shim sound)
    lib = rt.load_library()
    assert lib.nncase_hip_ctx_create(0, None) == -errno.EINVAL and classify(-errno.EINVAL)[0] == "errno"


def test_shim_calls_declared_entry_points_with_the_right_arity():
    header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    arity = {}
    for m in re.finditer(r"NNCASE_HIP_API\s+[\w\s\*]+?\b(nncase_hip_\w+)\s*\((.*?)\)\s*;", header, re.S):
        args = m.group(2).strip()
        arity[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1

    def call_args(text, start):
        """Top-level argument count of the call whose '(' is at `start`."""
        depth, count, i, seen = 0, 0, start, False
        while True:
            ch = text[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
                if depth == 0:
                    return count + 1 if seen else 0
            elif ch == "," and depth == 1:
                count += 1
            elif depth >= 1 and not ch.isspace():
                seen = True
            i += 1

    calls = 0
    for fname, text in shim_sources().items():
        code = re.sub(r"/\*.*?\*/", lambda m: " " * len(m.group(0)), text, flags=re.S)
        code = re.sub(r"//[^\n]*", lambda m: " " * len(m.group(0)), code)
        for m in re.finditer(r"\b(nncase_hip_\w+)\s*\(", code):
            name = m.group(1)
            if name.endswith("_t"):
                continue
            assert name in arity, f"{fname}: {name} is not declared in nncase_hip.h"
            assert call_args(code, m.end() - 1) == arity[name], f"{fname}: {name}"
            calls += 1
    assert calls >= 8
