"""OCP FP8 E4M3FN codec written from the format definition (numpy only).

TEST INFRASTRUCTURE: this file is part of the CPU oracle. Only tests, the
smoke check and the bench's cpu_baseline leg may import it; the product
package never does.

Format (OCP 8-bit Floating Point Specification, E4M3 "fn" flavour):
  bit 7 sign, bits 6..3 exponent (bias 7), bits 2..0 mantissa.
  exponent 0         -> subnormal, value = m * 2**-9           (m in 0..7)
  exponent 1..15     -> normal,   value = (1 + m/8) * 2**(e-7)
  code 0x7F / 0xFF   -> NaN (there is no infinity); largest finite = 0x7E = 448.

`encode_rne` rounds an fp32 value to nearest, ties to even, in the *unbounded*
exponent range and then maps anything that rounded above 448 to NaN.  That is
the non-saturating cast (what `tensor.to(torch.float8_e4m3fn)` does on a CPU);
`encode_rne_sat` clamps to +-448 first (the `satfinite` cast a GPU store
performs, cf. the implicit cast in the reference's `tl.store` to an fp8 pointer,
/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:112).

Nothing here calls torch, so the torch cast and this codec pin each other.
"""
import numpy as np

E4M3_MAX = 448.0


def decode_table() -> np.ndarray:
    """float32[256]: value of every e4m3fn code (NaN for 0x7F and 0xFF)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            v = float("nan")
        elif e == 0:
            v = sign * m * 2.0 ** -9
        else:
            v = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[code] = v
    return out


_DECODE = decode_table()


def decode(codes: np.ndarray) -> np.ndarray:
    """uint8 codes -> float32 values."""
    return _DECODE[np.asarray(codes, dtype=np.uint8)]


def encode_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> uint8 e4m3fn codes; round-to-nearest-even, overflow -> NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    out = np.empty(x.shape, dtype=np.uint8)

    nan_or_inf = mag >= np.uint32(0x7F800000)
    # 2**-6 == smallest normal e4m3 == float32 bits 0x3C800000
    small = mag < np.uint32(0x3C800000)

    # --- subnormal range: value/2**-9 rounded half-even to an integer 0..8.
    # (8 is code 0b0001000 = 2**-6, so the carry into the normal range is free.)
    ax = np.abs(x.astype(np.float64))
    sub_code = np.rint(ax * 512.0)  # np.rint is round-half-even; product exact in f64
    sub_code = np.where(small, sub_code, 0).astype(np.uint8)

    # --- normal range: keep 3 mantissa bits of the fp32 pattern, RNE on bit 20.
    lsb = (mag >> 20) & np.uint32(1)
    rounded = (mag.astype(np.uint64) + np.uint64(0x7FFFF) + lsb.astype(np.uint64)) & np.uint64(0xFFF00000)
    e32 = (rounded >> np.uint64(23)).astype(np.int64) - 127  # unbiased exponent
    m3 = ((rounded >> np.uint64(20)) & np.uint64(7)).astype(np.int64)
    norm_code = ((e32 + 7) << 3) | m3
    overflow = norm_code > 0x7E  # rounded above 448 (0x7F would read as NaN anyway)
    norm_code = np.where(overflow, 0x7F, norm_code)
    norm_code = np.clip(norm_code, 0, 0x7F).astype(np.uint8)

    out[...] = np.where(small, sub_code, norm_code)
    out[nan_or_inf] = 0x7F
    return out | sign


def encode_rne_sat(x: np.ndarray) -> np.ndarray:
    """float32 -> uint8 e4m3fn codes; finite values saturate at +-448; NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    clamped = np.where(np.isnan(x), x, np.clip(x, np.float32(-E4M3_MAX), np.float32(E4M3_MAX)))
    return encode_rne(clamped.astype(np.float32))


def bf16_bits_to_f32(u16: np.ndarray) -> np.ndarray:
    """uint16 bfloat16 patterns -> float32 (exact)."""
    return (np.asarray(u16, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> uint16 bfloat16 patterns, round-to-nearest-even, NaN kept quiet."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    lsb = (bits >> np.uint64(16)) & np.uint64(1)
    r = ((bits + np.uint64(0x7FFF) + lsb) >> np.uint64(16)).astype(np.uint16)
    nan = np.isnan(x)
    r[nan] = ((bits[nan] >> np.uint64(16)).astype(np.uint16)) | np.uint16(0x0040)
    return r


# ---------------------------------------------------------------------------
# OCP FP8 E5M2: bit 7 sign, bits 6..2 exponent (bias 15), bits 1..0 mantissa; IEEE-like (the top byte of a binary16):
#   exponent 0 -> subnormal, value = m * 2**-16; exponent 1..30 -> (1 + m/4) * 2**(e-15); exponent 31 -> inf (m = 0) / NaN.
#   largest finite = 0x7B = 57344.
# ---------------------------------------------------------------------------
E5M2_MAX = 57344.0


def decode_table_e5m2() -> np.ndarray:
    """float32[256]: value of every e5m2 code."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 2) & 0x1F
        m = code & 0x3
        if e == 0x1F:
            v = sign * float("inf") if m == 0 else float("nan")
        elif e == 0:
            v = sign * m * 2.0 ** -16
        else:
            v = sign * (1.0 + m / 4.0) * 2.0 ** (e - 15)
        out[code] = v
    return out


_DECODE_E5M2 = decode_table_e5m2()


def decode_e5m2(codes: np.ndarray) -> np.ndarray:
    return _DECODE_E5M2[np.asarray(codes, dtype=np.uint8)]


def encode_rne_e5m2(x: np.ndarray) -> np.ndarray:
    """float32 -> uint8 e5m2 codes; round-to-nearest-even, overflow -> inf, NaN -> 0x7F (sign kept)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    out = np.empty(x.shape, dtype=np.uint8)
    is_nan = mag > np.uint32(0x7F800000)
    small = mag < np.uint32(0x38800000)            # 2**-14, the smallest normal e5m2
    ax = np.abs(x.astype(np.float64))
    sub_code = np.where(small, np.rint(ax * 65536.0), 0).astype(np.uint8)     # m = value / 2**-16, half-even; 4 carries into e = 1
    lsb = (mag >> 21) & np.uint32(1)
    rounded = (mag.astype(np.uint64) + np.uint64(0xFFFFF) + lsb.astype(np.uint64)) & np.uint64(0xFFE00000)
    e32 = (rounded >> np.uint64(23)).astype(np.int64) - 127
    m2 = ((rounded >> np.uint64(21)) & np.uint64(3)).astype(np.int64)
    norm_code = ((e32 + 15) << 2) | m2
    norm_code = np.where(norm_code >= 0x7C, 0x7C, norm_code)                  # rounded above 57344 (or was inf): inf
    norm_code = np.clip(norm_code, 0, 0x7C).astype(np.uint8)
    out[...] = np.where(small, sub_code, norm_code)
    out[is_nan] = 0x7F
    return out | sign
