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
    assert C.sizeof(rt.Conv2dArgs) == 11 * 4 + 8 + 8 + 3 * 4 + 8 + 8 + 8 + 2 * 4
    assert C.sizeof(rt.MatmulArgs) == 4 + 8 + 8 + 3 * 4
    assert C.sizeof(rt.QBlockDesc) == 3 * 4 + 3 * 8 and C.sizeof(rt.QBlockArgs) == 8 * 4 + 4 * 8 + 6 * 4 + 4 + 8 + 2 * 4
    assert C.sizeof(rt.PagedAttnArgs) == 10 * 4
