"""Builds libdeepbind_hip.so for gfx950 with hipcc, in-tree next to this file.

    python -m deepbind_amd.build          # compile every csrc/*.hip and link

hipcc cross-compiles without a GPU present, so this runs anywhere the ROCm toolchain is installed.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libdeepbind_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-ffp-contract=off",                    # no silent fused multiply-adds: results are compared bit-for-bit where orders match
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # never emit packed-FP32 VALU instructions
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


# The running max of the k-mer kernel must compile to bare v_max / v_max3 instructions; with NaNs
# honoured every fmaxf gets two extra canonicalising ops. Infinities stay honoured (-inf seeds the max).
EXTRA = {"scanpool_kmer.hip": ["-fno-honor-nans"]}


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + EXTRA.get(os.path.basename(src), []) + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    jobs = jobs or min(8, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    if verbose:
        for obj, out in results:
            if out.strip():
                print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s" % res.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
