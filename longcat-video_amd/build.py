"""Builds the gfx950 engine into longcat_video_amd/lib/libbsa_mi355x.so.

    python longcat-video_amd/build.py [--keep-temps]

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm
toolchain is installed.  The library is built in-tree; nothing is installed.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "longcat_video_amd", "lib")
LIB = os.path.join(OUT_DIR, "libbsa_mi355x.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["bsa_capi.hip", "bsa_permute.hip", "bsa_select.hip", "bsa_fwd.hip", "bsa_fwd_frag.hip", "bsa_bwd.hip", "bsa_glue.hip", "bsa_gemm.hip"]
# The attention kernel never produces a NaN by construction (the -inf cases are guarded), so its
# maxima need no NaN-quieting extra instructions.  Infinities keep their IEEE meaning.
# The glue kernels restate eager fp32 expressions (x * cos + rot * sin, x * (scale + 1) + shift, x + gate * y)
# whose products and sums are rounded one by one: no contraction into FMAs there (explicit fmaf stays an FMA).
# The fragment pass and the GEMM epilogue share those expressions (bsa_rope.h) beside code that wants its FMAs:
# contraction stays on for the file and the shared functions switch it off with a pragma, which the compiler only
# honours under fast-honor-pragmas.
EXTRA_FLAGS = {"bsa_fwd.hip": ["-fno-honor-nans"], "bsa_fwd_frag.hip": ["-fno-honor-nans", "-ffp-contract=fast-honor-pragmas"],
               "bsa_bwd.hip": ["-fno-honor-nans"], "bsa_glue.hip": ["-ffp-contract=off"],
               "bsa_gemm.hip": ["-ffp-contract=fast-honor-pragmas"]}

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of generated code on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the engine cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(keep_temps: bool = False, verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    cc = hipcc()
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        cmd = [cc, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if keep_temps:
            cmd += ["-save-temps=obj"]
        out = _run(cmd)
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, len(sources))) as ex:
        objs = list(ex.map(compile_one, sources))
    _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-lhipblaslt"])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--keep-temps", action="store_true", help="keep the device assembly next to the objects")
    args = ap.parse_args()
    try:
        build(args.keep_temps)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
