"""Builds libmi355_layer.so (gfx950 only) from the HIP sources in this directory.

Usage: python -m scaling_amd.csrc.build      (or scaling_amd.csrc.build.build() from Python)
Each .hip file is one translation unit; objects go to ./build/, the library next to the sources.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libmi355_layer.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["abi.hip", "rmsnorm.hip", "swiglu.hip", "rotary.hip", "attn_host.hip", "attn_fwd.hip", "attn_bwd.hip",
           "attn_decode.hip", "attn_f32.hip", "cross_entropy.hip"]
F16_SOURCES = ["attn_fwd.hip", "attn_bwd.hip", "attn_decode.hip"]
# packed fp32 VALU instructions stay disabled for every device translation unit; the kernels never
# produce NaNs on purpose (masked scores are -inf and every inf - inf is guarded), so NaN-preserving
# canonicalisation of the MFMA results before max / min is switched off
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-fno-honor-nans", "-Wno-unused-command-line-argument"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libmi355_layer.so cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr))
    return proc


def build(verbose: bool = False, jobs: int = 8) -> str:
    hipcc = _hipcc()
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)

    def compile_one(job):
        src, suffix, defines = job
        obj = os.path.join(obj_dir, src.replace(".hip", suffix + ".o"))
        _run([hipcc] + FLAGS + defines + ["-c", src, "-o", obj])
        if verbose:
            print("compiled", src, " ".join(defines), flush=True)
        return obj

    # the attention kernels exist once per element type: bfloat16 (as is) and float16 (-DMI_ELEM_F16)
    jobs_list = [(s, "", []) for s in SOURCES] + [(s, "_f16", ["-DMI_ELEM_F16"]) for s in F16_SOURCES]
    jobs_list.sort(key=lambda j: 0 if j[0] in ("attn_fwd.hip", "attn_bwd.hip") else 1)   # the slow ones first
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, jobs_list))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("linked", LIB_PATH, flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
