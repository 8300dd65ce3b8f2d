"""Build libmdyfp8.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m mdy_triton_amd.csrc.build   (or call build())
The library lands next to this file so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["api.hip", "act_quant.hip", "weight_quant.hip", "quant_transpose.hip", "swiglu.hip", "weight_dequant.hip", "fp8_gemm.hip", "fp8_gemm_rowscaled.hip", "group_pad.hip", "add_bias.hip"]
LIB = os.path.join(HERE, "libmdyfp8.so")
# timing probes (ablated copies of the tile kernel, copy-only and MFMA-only ceilings): a library of its own that only
# bench.py's diagnostic modes load
PROBE_SOURCES = ["gemm_probe.hip", "ceiling_probe.hip"]
PROBE_LIB = os.path.join(HERE, "libmdyfp8_probe.so")

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32.
# No fast-math: the quantizers rely on IEEE division and uncontracted FMAs.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go to plain VGPRs: the GEMM folds them with v_fma_f32, which cannot read AGPRs
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose: bool = False) -> str:
    """Compile every source and link the shared library; returns its path."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]
    probe_objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in PROBE_SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc, *HIPCC_FLAGS, "-c", os.path.join(HERE, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=8) as ex:
        for out in ex.map(compile_one, zip(SOURCES + PROBE_SOURCES, objs + probe_objs)):
            if verbose and out.strip():
                print(out)
    tmp = LIB + ".tmp"
    out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB)
    tmp = PROBE_LIB + ".tmp"
    out += _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *probe_objs])
    os.replace(tmp, PROBE_LIB)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
