"""Pins the fp32 -> e4m3fn cast: the from-definition codec (oracle/fp8_format.py)
against torch's CPU cast, on every code, every rounding midpoint and its fp32
neighbours, the subnormal grid, the overflow edge and the specials."""
import numpy as np
import torch

from oracle import fp8_format as F


def _neighbours(v: np.ndarray) -> np.ndarray:
    v = v.astype(np.float32)
    return np.concatenate([v, np.nextafter(v, np.float32(np.inf)), np.nextafter(v, np.float32(-np.inf))])


def _torch_cast(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_decode_table_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    tab = F.decode_table()
    assert np.array_equal(np.isnan(ref), np.isnan(tab))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok].view(np.uint32), tab[ok].view(np.uint32))
    assert tab[0x7E] == 448.0 and tab[0x01] == 2.0 ** -9 and tab[0x08] == 2.0 ** -6
    assert np.isnan(tab[0x7F]) and np.isnan(tab[0xFF])


def test_every_code_round_trips():
    tab = F.decode_table()
    finite = ~np.isnan(tab)
    codes = np.arange(256, dtype=np.uint8)[finite]
    assert np.array_equal(F.encode_rne(tab[finite]), codes)
    assert np.array_equal(_torch_cast(tab[finite]), codes)


def test_midpoints_and_neighbours_tie_to_even():
    tab = F.decode_table()
    pos = np.sort(tab[:0x7F])  # 0 .. 448
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    # midpoints are exact in fp32; ties go to the even code
    got = F.encode_rne(mids)
    lo = np.arange(0, 0x7E, dtype=np.uint8)
    expect = np.where(lo % 2 == 0, lo, lo + 1).astype(np.uint8)
    assert np.array_equal(got, expect)
    pts = _neighbours(np.concatenate([mids, pos, -mids, -pos]))
    assert np.array_equal(F.encode_rne(pts), _torch_cast(pts))


def test_overflow_edge_and_specials():
    x = np.array([448.0, 463.99997, 464.0, 464.00003, 465.0, 480.0, 1e4, 3e38, np.inf, -np.inf, np.nan,
                  -448.0, -464.0, -465.0, 0.0, -0.0, 2.0 ** -10, np.nextafter(np.float32(2.0 ** -10), np.float32(1)),
                  -(2.0 ** -10), 1e-30, -1e-30, 1e-45], dtype=np.float32)
    got = F.encode_rne(x)
    ref = _torch_cast(x)
    # NaN payload sign is not part of the contract
    nan = (ref & 0x7F) == 0x7F
    assert np.array_equal((got & 0x7F) == 0x7F, nan)
    assert np.array_equal(got[~nan], ref[~nan])
    assert got[0] == 0x7E and got[2] == 0x7E and (got[4] & 0x7F) == 0x7F
    assert got[14] == 0x00 and got[15] == 0x80
    assert got[16] == 0x00 and got[17] == 0x01 and got[18] == 0x80   # 2**-10 ties to even (zero)
    sat = F.encode_rne_sat(x)
    assert sat[4] == 0x7E and sat[6] == 0x7E and sat[8] == 0x7E and sat[9] == 0xFE and (sat[10] & 0x7F) == 0x7F


def test_random_bits_match_torch():
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[np.isfinite(x)]
    # concentrate half of the samples in the representable range
    y = (rng.standard_normal(1 << 20) * rng.choice([1e-3, 1.0, 100.0, 400.0], size=1 << 20)).astype(np.float32)
    for v in (x, y):
        got, ref = F.encode_rne(v), _torch_cast(v)
        nan = (ref & 0x7F) == 0x7F
        assert np.array_equal((got & 0x7F) == 0x7F, nan)
        assert np.array_equal(got[~nan], ref[~nan])


def test_bf16_helpers():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(100000).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(F.f32_to_bf16_bits_rne(x), ref)
    assert np.array_equal(F.bf16_bits_to_f32(ref), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def test_e5m2_codec_against_torch_cpu_cast():
    """The from-definition e5m2 codec (the top byte of a binary16: 5 exponent bits, 2 mantissa bits, inf and NaN) and
    torch's CPU cast pin each other: every code decodes alike, and every rounding midpoint with its fp32 neighbours,
    the subnormal grid, the overflow edge (57344 | 61440 rounds to inf), signed zeros, inf and NaN encode alike."""
    codes = np.arange(256, dtype=np.uint8)
    vals = F.decode_e5m2(codes)
    tvals = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    assert np.array_equal(np.isnan(vals), np.isnan(tvals)) and np.array_equal(vals[~np.isnan(vals)], tvals[~np.isnan(tvals)])
    finite = np.sort(vals[np.isfinite(vals) & (vals >= 0)])
    mids = (finite[:-1].astype(np.float64) + finite[1:].astype(np.float64)) / 2
    pts = []
    for v in np.concatenate([finite.astype(np.float64), mids]):
        f = np.float32(v)
        pts += [f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))]
    pts += [57344.0, 61439.0, 61440.0, 61441.0, 65536.0, 1e30, 2.0 ** -16, 2.0 ** -17, 1.5 * 2.0 ** -17, 2.0 ** -18, np.inf]
    x = np.array(pts, dtype=np.float32)
    x = np.concatenate([x, -x, np.array([np.nan], dtype=np.float32)])
    rng = np.random.default_rng(3)
    x = np.concatenate([x, (rng.standard_normal(500000) * 10.0 ** rng.integers(-6, 5, 500000)).astype(np.float32)])
    mine = F.encode_rne_e5m2(x)
    theirs = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    nan = np.isnan(x)
    assert np.array_equal(mine[~nan], theirs[~nan])
    assert np.all((mine[nan] & 0x7F) > 0x7C) and np.all((theirs[nan] & 0x7F) > 0x7C)
    # round trip: every finite code encodes to itself
    back = F.encode_rne_e5m2(vals[np.isfinite(vals)])
    assert np.array_equal(back, codes[np.isfinite(vals)])
