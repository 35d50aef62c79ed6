"""Builds libm2_amd.so (gfx950) from m2_amd/csrc with hipcc, in-tree.

    python m2_amd/build.py                 # compile every .hip and link
    python m2_amd/build.py --incremental   # recompile only the sources that changed
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libm2_amd.so")
SOURCES = ["common.hip", "fftconv_kernels.hip", "fftconv_real_kernels.hip", "fftconv_split_kernels.hip", "hyena_filter_kernels.hip", "filter_fused_kernels.hip", "blockdiag_kernels.hip", "wo_layernorm_kernels.hip",
           "mlp_fused_kernels.hip", "glu_stream_kernels.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU instructions are switched off on purpose (device flag, the host pass warns about it)
FLAGS = ["-std=c++17", "-O3", "--offload-arch=gfx950", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _up_to_date(obj: str) -> bool:
    if not os.path.exists(obj):
        return False
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps += [os.path.join(CSRC, os.path.splitext(os.path.basename(obj))[0] + ".hip"),
             os.path.join(HERE, "..", "include", "m2_amd.h"), os.path.abspath(__file__)]
    return all(os.path.getmtime(d) < t for d in deps)


def _compile(src: str, incremental: bool = False) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    if incremental and _up_to_date(obj):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, incremental: bool = False) -> str:
    """Compiles every source (or, with incremental=True, only those older than their .hip / headers) and links."""
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda src: _compile(src, incremental), SOURCES))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
