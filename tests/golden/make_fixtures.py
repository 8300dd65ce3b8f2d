"""Writes the small closed-form fixtures under tests/golden/ (run from the repo root:
`python tests/golden/make_fixtures.py`).

Nothing here runs the oracle's quantizer or any reference code: every expected
output follows from the e4m3fn format definition (oracle/fp8_format.decode_table)
and exact power-of-two scaling, so the fixtures pin the oracle and the kernels
from outside.

act_quant_codes.npz
    x_bits  uint16 [R, 256]  bfloat16 patterns, two 128-groups per row
    y       uint8  [R, 256]  expected e4m3fn bytes
    s       float32 [R, 2]   expected scales
    Row r, group g holds every finite e4m3fn value of one sign half (codes
    0x00..0x7E or 0x80..0xFE, 127 values + one extra 448) multiplied by 2**e(r,g).
    All those products are exact in bfloat16, the group's absmax is 448 * 2**e, so
    the scale is exactly 2**e (official dialect) and x / s is exactly the e4m3fn
    value: the expected byte is the code itself.
weight_dequant_codes.npz
    x uint8 [128, 256] all codes, s float32 [1, 2] = (1.0, 2**-5):
    expected bf16 patterns are decode(code) * s, exact in bfloat16.
gemm_exact.npz
    small-integer e4m3fn operands with power-of-two scales whose products and
    sums are exact in fp32 and in bf16; the expected output is computed in int64.
act_quant_block_e5m2.npz
    the same construction as act_quant_codes.npz for the e5m2 format (the default dtype of
    deepseekv3/fp8_kernel.py's act_quant_block) in BOTH directions: x_bits uint16 [128, 256]
    bfloat16 patterns; column c of the 128 rows holds every finite non-negative or non-positive
    e5m2 value (codes 0x00..0x7B or 0x80..0xFB, 124 values, plus four more copies of 57344)
    times 2**e(c), so the transposed quantization (along the rows) must return the codes
    themselves: y_t uint8 [256, 128], s_t float32 [256, 1] = 2**e(c).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle.fp8_format import decode_table, decode_table_e5m2, f32_to_bf16_bits_rne  # noqa: E402


def bf16_bits_exact(x32: np.ndarray) -> np.ndarray:
    bits = x32.astype(np.float32).view(np.uint32)
    assert np.all((bits & 0xFFFF) == 0), "value not exact in bfloat16"
    return (bits >> 16).astype(np.uint16)


def make_act_quant_codes():
    tab = decode_table()
    exps = [0, -3, 5, -20, 17, 1, -9, 30]
    R = len(exps) // 2
    x_bits = np.zeros((R, 256), np.uint16)
    y = np.zeros((R, 256), np.uint8)
    s = np.zeros((R, 2), np.float32)
    rng = np.random.default_rng(1234)
    for r in range(R):
        for g in range(2):
            e = exps[2 * r + g]
            base = 0x80 if (r + g) % 2 else 0x00
            codes = np.concatenate([np.arange(base, base + 0x7F), [base + 0x7E]]).astype(np.uint8)
            rng.shuffle(codes)
            vals = tab[codes].astype(np.float64) * 2.0 ** e
            x_bits[r, 128 * g:128 * (g + 1)] = bf16_bits_exact(vals.astype(np.float32))
            y[r, 128 * g:128 * (g + 1)] = codes
            s[r, g] = np.float32(2.0 ** e)
    np.savez(os.path.join(HERE, "act_quant_codes.npz"), x_bits=x_bits, y=y, s=s)


def make_weight_dequant_codes():
    tab = decode_table()
    x = np.tile(np.arange(256, dtype=np.uint8), (128, 1))
    s = np.array([[1.0, 2.0 ** -5]], np.float32)
    finite = ~np.isnan(tab)
    exp = np.zeros((128, 256), np.float32)
    exp[:, :128] = tab[:128][None, :] * s[0, 0]
    exp[:, 128:] = tab[128:][None, :] * s[0, 1]
    y_bits = np.zeros((128, 256), np.uint16)
    y_bits[:, finite] = bf16_bits_exact(np.where(np.isnan(exp), 0, exp)[:, finite])
    np.savez(os.path.join(HERE, "weight_dequant_codes.npz"), x=x, s=s, y_bits=y_bits, finite=finite)


def make_gemm_exact():
    tab = decode_table()
    rng = np.random.default_rng(99)
    M, N, K = 48, 272, 384
    # integer-valued codes: -4..4
    ints = np.arange(-4, 5)
    code_of = {int(v): int(np.where(tab == np.float32(v))[0][0]) for v in ints}
    code_of[0] = 0
    ai = rng.integers(-4, 5, size=(M, K))
    bi = rng.integers(-4, 5, size=(N, K))
    a = np.vectorize(code_of.get)(ai).astype(np.uint8)
    b = np.vectorize(code_of.get)(bi).astype(np.uint8)
    KB, NB = K // 128, (N + 127) // 128
    a_e = rng.integers(-2, 3, size=(M, KB))
    b_e = rng.integers(-2, 3, size=(NB, KB))
    a_s = (2.0 ** a_e).astype(np.float32)
    b_s = (2.0 ** b_e).astype(np.float32)
    # exact result in integers scaled by 2**8 (scales are >= 2**-4 combined)
    c = np.zeros((M, N), np.int64)
    for kb in range(KB):
        part = ai[:, kb * 128:(kb + 1) * 128] @ bi[:, kb * 128:(kb + 1) * 128].T
        sc = (2 ** (a_e[:, kb][:, None] + b_e[np.arange(N) // 128, kb][None, :] + 4)).astype(np.int64)
        c += part * sc
    c = c.astype(np.float64) / 16.0
    # representable in bf16?  keep only a fixture where every entry is (|c| small integers / 16 with <= 8 significant bits)
    c32 = c.astype(np.float32)
    bits = f32_to_bf16_bits_rne(c32)
    exact = (c32.view(np.uint32) & 0xFFFF) == 0
    np.savez(os.path.join(HERE, "gemm_exact.npz"), a=a, b=b, a_s=a_s, b_s=b_s, c_f32=c32, c_bf16_bits=bits,
             bf16_exact=exact)


def make_act_quant_block_e5m2():
    tab = decode_table_e5m2()
    rng = np.random.default_rng(77)
    R, C = 128, 256
    x_bits = np.zeros((R, C), np.uint16)
    y_t = np.zeros((C, R), np.uint8)
    s_t = np.zeros((C, 1), np.float32)
    for c in range(C):
        e = int(rng.integers(-20, 21))
        base = 0x80 if c % 2 else 0x00
        codes = np.concatenate([np.arange(base, base + 0x7C), [base + 0x7B] * 4]).astype(np.uint8)   # 124 finite codes + 57344 x 4
        rng.shuffle(codes)
        vals = tab[codes].astype(np.float64) * 2.0 ** e
        x_bits[:, c] = bf16_bits_exact(vals.astype(np.float32))     # e5m2 values (2 mantissa bits) are exact in bfloat16
        y_t[c] = codes
        s_t[c, 0] = np.float32(2.0 ** e)
    np.savez(os.path.join(HERE, "act_quant_block_e5m2.npz"), x_bits=x_bits, y_t=y_t, s_t=s_t)


if __name__ == "__main__":
    make_act_quant_block_e5m2()
    make_act_quant_codes()
    make_weight_dequant_codes()
    make_gemm_exact()
    print("fixtures written to", HERE)
