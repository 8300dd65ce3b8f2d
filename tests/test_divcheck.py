"""Runs the exhaustive CPU proof (oracle/divcheck.c) that the quantizers'
reciprocal + 2-FMA quotient gives the same e4m3fn byte as IEEE division for
every (amax, x) pair of bfloat16 values, and checks that the exponent range
hard-coded in the kernels is the proven one."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_fast_quotient_proof_and_kernel_constant():
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-s"], check=True)
    out = subprocess.run([os.path.join(ROOT, "oracle", "_build", "divcheck")], check=True,
                         stdout=subprocess.PIPE, text=True).stdout
    clean = {int(m.group(1)): (int(m.group(2)), int(m.group(3)))
             for m in re.finditer(r"mode (\d) clean_amax_exp_range (-?\d+) (-?\d+)", out)}
    fp8_bad = {int(m.group(1)): int(m.group(2))
               for m in re.finditer(r"mode (\d) pairs \d+ f32_mismatch \d+ fp8_mismatch (\d+)", out)}
    # DeepLinear dialect: clean for every finite amax
    assert fp8_bad[1] == 0 and clean[1] == (0, 254)
    # official dialect: clean from biased exponent 23 up (below, s = amax/448 is subnormal or the residual underflows)
    assert clean[0][1] == 254
    src = open(os.path.join(ROOT, "mdy_triton_amd", "csrc", "common.h")).read()
    k = int(re.search(r"kFastQuotientMinExp\s*=\s*(\d+)", src).group(1))
    assert k >= clean[0][0], "kernel uses the fast quotient outside the proven range"
    assert k == 23
