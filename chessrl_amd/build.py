"""Build libchessrl_amd.so in-tree with hipcc for gfx950.

Each translation unit is compiled to an object in parallel, then linked into
chessrl_amd/libchessrl_amd.so. Run as ``python -m chessrl_amd.build``.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libchessrl_amd.so")

SOURCES = [
    "host/chess.cpp",
    "kernels/gemm.hip",
    "kernels/gemm_dma.hip",
    "kernels/gemm_dma_resnorm.hip",
    "kernels/gemm_sp2.hip",
    "kernels/gemm_dmaf.hip",
    "kernels/gemm_dmam.hip",
    "kernels/gemm_shortk.hip",
    "kernels/norm_embed.hip",
    "kernels/attention.hip",
    "kernels/heads.hip",
    "kernels/probe.hip",
    "kernels/decode.hip",
    "model.hip",
    "api.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-pass-failed",
]


def _compile(src):
    obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    return obj


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    # -shared lets unresolved names through to load time: a kernel whose host stub the compiler dropped shows up here.
    nm = subprocess.run(["nm", "-u", LIB], capture_output=True, text=True)
    missing = [l.split()[-1] for l in nm.stdout.splitlines() if "_ZN3crl" in l]
    if missing:
        raise RuntimeError("unresolved symbols of this library's own namespace:\n" + "\n".join(missing))
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
