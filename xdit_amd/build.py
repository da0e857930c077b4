"""Build the HIP shared library of the attention hot path for gfx950 (in-tree, with hipcc).

`python -m xdit_amd.build` compiles `xdit_amd/csrc/*.hip` into
`xdit_amd/libxdit_amd_attn.so`.  hipcc cross-compiles for gfx950 without a GPU present.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJDIR = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libxdit_amd_attn.so")
SOURCES = ["api.hip", "attn_fwd_16.hip", "attn_fwd_16_ring.hip", "attn_fwd_fp8.hip", "attn_fwd_f32.hip", "lse_merge.hip", "fp8_quant.hip", "qk_prologue.hip"]
FLAGS = [
    # an atomic under a one-lane branch stays one plain atomic whose result is awaited where it is used
    "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


# per-file additions; the prologue reproduces separately rounded fp32 products and sums
EXTRA_FLAGS = {"qk_prologue.hip": ["-ffp-contract=off"]}


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build(verbose=True):
    """Compile every HIP source and link the shared library. Always recompiles."""
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
