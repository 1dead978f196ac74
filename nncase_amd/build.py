"""Compiles libnncase_hip.so (gfx950 only) in-tree with hipcc.

    python -m nncase_amd.build            # rebuild everything
Each .hip file is compiled to an object in parallel and the objects are linked
into nncase_amd/lib/libnncase_hip.so.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libnncase_hip.so")

SOURCES = ["ctx.hip", "quant.hip", "qconv.hip", "qconv_igemm.hip", "qconv_igemm_rows16.hip", "qconv_igemm_rows8.hip", "qconv_igemm_vec16.hip",
           "qconv_igemm_vec8.hip", "qconv_igemm_vec4.hip", "qconv_igemm_bytes.hip", "qconv_wide_rows16.hip", "qconv_wide_vec16.hip", "qblock.hip", "qpair.hip", "qconv_smallc.hip", "qconv_dw.hip", "layout.hip", "glue.hip", "attn.hip", "llm.hip", "function.hip", "kmodel.hip"]

# -ffp-contract=off / -fno-fast-math: every fp32 step of the requantisation must be a
# single IEEE operation.  packed-fp32-ops is switched off for the device pass.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libnncase_hip.so cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    # NNCASE_HIP_EXTRA_FLAGS: additional hipcc flags (e.g. -D switches of an experiment), space separated
    cmd = [hipcc(), *FLAGS, *os.environ.get("NNCASE_HIP_EXTRA_FLAGS", "").split(), "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    warn = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and "warning" in l)
    if warn:
        sys.stderr.write(f"[{src}] {warn}\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build()
