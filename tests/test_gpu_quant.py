"""GPU parity of the quantizers and the dequantizer against the CPU oracle:
e4m3fn bytes and fp32 scales bit-exact, dequantized bf16 bit-exact."""
import ctypes
import os

import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from mdy_triton_amd import _lib
from oracle import fp8_format as F
from oracle import oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
FP8 = torch.float8_e4m3fn
DEV = "cuda:0"


def u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def same_bytes_mod_nan(got, ref):
    """Bit-exact, except that the two NaN codes (0x7F / 0xFF) compare equal."""
    nan = (ref & 0x7F) == 0x7F
    return np.array_equal((got & 0x7F) == 0x7F, nan) and np.array_equal(got[~nan], ref[~nan])


def bf16_from_bits(bits):
    return torch.from_numpy(bits.astype(np.uint16).view(np.int16).copy()).view(torch.bfloat16)


# ------------------------------------------------------------------ the cast itself
def _device_cast(x: np.ndarray, saturate: int) -> np.ndarray:
    xt = torch.from_numpy(x.copy()).to(DEV)
    y = torch.empty(x.size, dtype=torch.uint8, device=DEV)
    _lib.check(_lib.load().mdy_cast_f32_to_e4m3(xt.data_ptr(), y.data_ptr(), x.size, saturate, None), "cast")
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_device_cast_matches_format_definition():
    tab = F.decode_table()
    pos = np.sort(tab[:0x7F])
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    pts = np.concatenate([pos, mids, -pos, -mids])
    pts = np.concatenate([pts, np.nextafter(pts, np.float32(np.inf)), np.nextafter(pts, np.float32(-np.inf))])
    rng = np.random.default_rng(0)
    rnd = (rng.standard_normal(1 << 18) * rng.choice([1e-3, 1.0, 100.0, 300.0], size=1 << 18)).astype(np.float32)
    rnd = rnd[np.abs(rnd) <= 448.0]
    x = np.concatenate([pts, rnd, np.array([448.00003, -448.00003, 0.0, -0.0, 1e-30, -1e-30], np.float32)])
    x = x[np.abs(x) < 464.0].astype(np.float32)
    assert np.array_equal(_device_cast(x, 0), F.encode_rne(x))
    # saturating flavour over the whole fp32 range, NaN kept
    big = np.array([464.0, 465.0, 1e4, 3e38, np.inf, -464.0, -1e9, -np.inf, np.nan, 500.0], np.float32)
    xs = np.concatenate([x, big])
    assert same_bytes_mod_nan(_device_cast(xs, 1), F.encode_rne_sat(xs))


def test_fast_quotient_equals_division_on_device():
    """Every bf16 amax x every bf16 |x| <= amax, both dialects, on the device's own
    divider and FMA: the byte (and where the fast path is taken, nothing else) agrees."""
    out = torch.zeros(4, dtype=torch.int64, device=DEV)
    for mode in (0, 1):
        _lib.check(_lib.load().mdy_quotient_selfcheck(out.data_ptr(), 0, 0x7F80, mode, None), "selfcheck")
        torch.cuda.synchronize()
        pairs, f32_bad, fp8_bad, plain = out.cpu().tolist()
        assert pairs == 1065402240
        assert fp8_bad == 0
        if mode == 0:
            assert plain < pairs // 8   # only tiny-amax groups divide plainly


# ------------------------------------------------------------------ act_quant (official dialect)
def test_act_quant_golden_codes():
    d = np.load(os.path.join(GOLD, "act_quant_codes.npz"))
    y, s = m.act_quant(bf16_from_bits(d["x_bits"]).to(DEV))
    assert np.array_equal(u8(y), d["y"])
    assert np.array_equal(s.cpu().numpy().view(np.uint32), d["s"].view(np.uint32))


@pytest.mark.parametrize("kind,M,K,seed", [
    ("normal", 128, 1024, 0), ("outliers", 4096, 7168, 1), ("normal", 4096, 7168, 2), ("heavy", 4096, 18432, 3),
    ("normal", 1, 2048, 4), ("normal", 16, 7168, 5), ("normal", 64, 2048, 6), ("normal", 3, 128, 7),
    ("normal", 37, 640, 8),
])
def test_act_quant_bit_exact(kind, M, K, seed):
    x = P.activations(kind, M, K, seed)
    y_ref, s_ref = O.act_quant(x)
    y, s = m.act_quant(x.to(DEV))
    assert y.dtype == FP8 and y.shape == x.shape and s.shape == (M, K // 128) and s.dtype == torch.float32
    assert torch.equal(s.cpu(), s_ref)
    assert np.array_equal(u8(y), u8(y_ref))


def test_act_quant_leading_dims_and_empty():
    x = P.activations("normal", 24, 256, 9).reshape(2, 3, 4, 256)
    y, s = m.act_quant(x.to(DEV))
    y_ref, s_ref = O.act_quant(x)
    assert y.shape == x.shape and s.shape == (2, 3, 4, 2)
    assert np.array_equal(u8(y), u8(y_ref)) and torch.equal(s.cpu(), s_ref)
    y0, s0 = m.act_quant(torch.empty(0, 256, dtype=torch.bfloat16, device=DEV))
    assert y0.shape == (0, 256) and s0.shape == (0, 2)


def test_act_quant_edge_values():
    """Tiny, subnormal, huge, signed-zero, all-zero, inf and NaN groups."""
    rng = np.random.default_rng(11)
    rows = []
    base = rng.standard_normal(128).astype(np.float32)
    for scale in (1.0, 2.0 ** -100, 2.0 ** -110, 2.0 ** -120, 2.0 ** -126, 2.0 ** -130, 2.0 ** 100, 2.0 ** 120, 3e38 / 4):
        rows.append(base * np.float32(scale))
    z = np.zeros(128, np.float32)
    rows.append(z.copy())                                   # all zero -> s = 0, y = NaN
    nz = z.copy(); nz[0] = 1.0; nz[1] = -0.0; nz[2] = 2.0 ** -133  # signed zero / flush-to-zero quotient
    rows.append(nz)
    inf = base.copy(); inf[5] = np.inf; inf[6] = -np.inf
    rows.append(inf)
    x = torch.from_numpy(np.stack(rows)).bfloat16()
    y_ref, s_ref = O.act_quant(x)
    y, s = m.act_quant(x.to(DEV))
    sr, sg = s_ref.numpy(), s.cpu().numpy()
    assert np.array_equal(np.isnan(sr), np.isnan(sg))
    assert np.array_equal(sr[~np.isnan(sr)].view(np.uint32), sg[~np.isnan(sg)].view(np.uint32))
    assert same_bytes_mod_nan(u8(y), u8(y_ref))
    assert np.all((u8(y)[9] & 0x7F) == 0x7F)
    assert u8(y)[10][1] == 0x80


def test_act_quant_nan_is_ignored_by_the_group_max():
    """A NaN element stays NaN; the rest of its group is quantized with the max of the
    finite values (the hardware max ignores NaN, as the reference's tl.max does)."""
    x = P.activations("normal", 2, 256, 12)
    x[0, 7] = float("nan")
    y, s = m.act_quant(x.to(DEV))
    xz = x.clone(); xz[0, 7] = 0.0
    y_ref, s_ref = O.act_quant(xz)
    assert torch.equal(s.cpu(), s_ref)
    got, ref = u8(y), u8(y_ref)
    assert (got[0, 7] & 0x7F) == 0x7F
    got[0, 7] = ref[0, 7]
    assert np.array_equal(got, ref)


# ------------------------------------------------------------------ quant_input (DeepLinear dialect)
@pytest.mark.parametrize("M,K,seed", [(128, 1024, 0), (4096, 7168, 1), (1, 2048, 2), (6, 300, 3), (37, 641, 4),
                                      (64, 7168, 5), (255, 384, 6)])
def test_quant_input_bit_exact(M, K, seed):
    x = P.activations("outliers", M, K, seed)
    y_ref, s_ref, _, _ = O.quant_input(x, True)
    y, s, y_t, s_t = m.quant_input(x.to(DEV), True)
    assert y_t is None and s_t is None
    assert y.shape == y_ref.shape and s.shape == s_ref.shape and s.stride() == s_ref.stride()
    assert torch.equal(s.cpu(), s_ref)
    assert np.array_equal(u8(y), u8(y_ref))


@pytest.mark.parametrize("M,K,seed", [(16384, 4096, 8), (8230, 8198, 9), (9001, 7552, 10)])
def test_quant_input_large_bit_exact(M, K, seed):
    """From 2^26 padded elements on, the forward quantizer runs 32-row blocks that stage the column-major
    scales in LDS; ragged M (padded to 4) and K (not a multiple of 8: scalar loads) included."""
    x = P.activations("outliers", M, K, seed)
    x[5, 3] = 3e4; x[M - 1, K - 1] = -2e4                                    # saturating groups
    y_ref, s_ref, _, _ = O.quant_input(x, True)
    y, s, _, _ = m.quant_input(x.to(DEV), True)
    assert y.shape == y_ref.shape and s.shape == s_ref.shape and s.stride() == s_ref.stride()
    assert y.shape[0] * y.shape[1] >= 1 << 26
    assert torch.equal(s.cpu(), s_ref)
    assert np.array_equal(u8(y), u8(y_ref))


def test_quant_input_strided_rows_and_saturation():
    big = P.activations("normal", 40, 1024, 7)
    x = big[:, 128:128 + 512]                      # row stride 1024, column stride 1, offset 256 bytes
    x[0, 0] = 3e4; x[0, 1] = -2e4; x[1, 3] = 1.5e4
    y_ref, s_ref, _, _ = O.quant_input(x, True)
    y, s, _, _ = m.quant_input(big.to(DEV)[:, 128:128 + 512], True)
    assert torch.equal(s.cpu(), s_ref) and np.array_equal(u8(y), u8(y_ref))
    xt = big.t()                                   # column stride != 1
    y_ref, s_ref, _, _ = O.quant_input(xt, True)
    y, s, _, _ = m.quant_input(big.to(DEV).t(), True)
    assert torch.equal(s.cpu(), s_ref) and np.array_equal(u8(y), u8(y_ref))


# ------------------------------------------------------------------ training-time quantizers
def _same_quant(got, ref):
    for g_, r_ in zip(got, ref):
        assert g_.shape == r_.shape and g_.stride() == r_.stride()
        if r_.dtype == FP8:
            assert np.array_equal(u8(g_), u8(r_))
        else:
            assert torch.equal(g_.cpu().contiguous(), r_.contiguous())


@pytest.mark.parametrize("M,K,seed", [(256, 256, 0), (512, 1024, 1), (130, 300, 2), (1, 7, 3), (4096, 7168, 4),
                                      (257, 129, 5)])
def test_quant_input_training_bit_exact(M, K, seed):
    x = P.activations("outliers", M, K, seed)
    _same_quant(m.quant_input(x.to(DEV), False), O.quant_input(x, False))


@pytest.mark.parametrize("M,N,seed", [(256, 256, 0), (1024, 512, 1), (130, 200, 2), (3, 5, 3), (4096, 1536, 4),
                                      (385, 127, 5)])
def test_quant_grad_output_bit_exact(M, N, seed):
    dy = P.activations("outliers", M, N, seed)
    _same_quant(m.quant_grad_output(dy.to(DEV)), O.quant_grad_output(dy))


def test_training_quantizers_strides_and_saturation():
    big = P.activations("normal", 300, 1024, 8)
    big[0, 130] = 3e4; big[5, 131] = -2e4; big[140, 700] = 1.5e4      # beyond the 1e4 clamp: plain division + saturation
    for view in (lambda t: t[:, 128:128 + 520], lambda t: t.t(), lambda t: t[::2, 1::3], lambda t: t[:1].expand(40, 1024)):
        x = view(big)
        for fn_g, fn_o in ((lambda t: m.quant_input(t, False), lambda t: O.quant_input(t, False)),
                           (m.quant_grad_output, O.quant_grad_output)):
            got, ref = fn_g(view(big.to(DEV))), fn_o(x)
            for g_, r_ in zip(got, ref):
                if r_.dtype == FP8:
                    assert np.array_equal(u8(g_), u8(r_))
                else:
                    assert torch.equal(g_.cpu().contiguous(), r_.contiguous())


def test_training_quantizers_ignore_nan_in_the_group_max():
    """As in the forward quantizer: a NaN element stays NaN in both copies, its row, column and block
    are scaled by the max of the finite values."""
    x = P.activations("normal", 256, 256, 13)
    x[3, 200] = float("nan")
    xz = x.clone(); xz[3, 200] = 0.0
    for fn_g, fn_o in ((lambda t: m.quant_input(t, False), lambda t: O.quant_input(t, False)),
                       (m.quant_grad_output, O.quant_grad_output)):
        (y, s, y_t, s_t), (y_r, s_r, yt_r, st_r) = fn_g(x.to(DEV)), fn_o(xz)
        assert torch.equal(s.cpu().contiguous(), s_r.contiguous()) and torch.equal(s_t.cpu().contiguous(), st_r.contiguous())
        got, got_t = u8(y), u8(y_t)
        assert (got[3, 200] & 0x7F) == 0x7F and (got_t[200, 3] & 0x7F) == 0x7F
        got[3, 200] = 0; got_t[200, 3] = 0
        assert np.array_equal(got, u8(y_r)) and np.array_equal(got_t, u8(yt_r))


def test_quant_transpose_abi_rejects_bad_arguments():
    L = _lib.load()
    x = torch.zeros(256, 256, dtype=torch.bfloat16, device=DEV)
    y = torch.empty(256, 256, dtype=torch.uint8, device=DEV)
    s = torch.empty(2, 256, dtype=torch.float32, device=DEV)
    args = lambda **kw: [kw.get("x", x.data_ptr()), kw.get("y", y.data_ptr()), s.data_ptr(), kw.get("y_t", y.data_ptr()),
                         s.data_ptr(), 256, 256, 256, 1, kw.get("PM", 256), kw.get("PK", 256), kw.get("skb", 256), kw.get("t_mode", 0), None]
    assert L.mdy_quant_transpose(*args(t_mode=2)) == -4
    assert L.mdy_quant_transpose(*args(PM=200)) == -2
    assert L.mdy_quant_transpose(*args(PK=384 + 64)) == -2
    assert L.mdy_quant_transpose(*args(y_t=None)) == -1
    assert L.mdy_quant_transpose(*args(skb=100)) == -2
    assert L.mdy_quant_transpose(*args(y=y.data_ptr() + 4)) == -3


# ------------------------------------------------------------------ quant_weight
@pytest.mark.parametrize("N,K,only_forward,seed", [(1024, 1024, True, 0), (1536, 7168, True, 1), (200, 300, True, 2),
                                                   (200, 300, False, 3), (512, 256, False, 4), (129, 257, False, 5)])
def test_quant_weight_bit_exact(N, K, only_forward, seed):
    w = P.weights_bf16(N, K, seed)
    ref = O.quant_weight(w, only_forward)
    got = m.quant_weight(w.to(DEV), only_forward)
    for r, g in zip(ref, got):
        if r is None:
            assert g is None
            continue
        assert g.shape == r.shape
        if r.dtype == FP8:
            assert np.array_equal(u8(g), u8(r))
        else:
            assert torch.equal(g.cpu(), r)


def test_quant_weight_transposed_view_input():
    w, _, _ = P.weights(256, 384, 6)
    ref = O.quant_weight(w.t(), True)
    got = m.quant_weight(w.to(DEV).t(), True)
    assert np.array_equal(u8(got[0]), u8(ref[0])) and torch.equal(got[1].cpu(), ref[1])


# ------------------------------------------------------------------ weight_dequant
def test_weight_dequant_golden_codes():
    d = np.load(os.path.join(GOLD, "weight_dequant_codes.npz"))
    x = torch.from_numpy(d["x"]).view(FP8).to(DEV)
    y = m.weight_dequant(x, torch.from_numpy(d["s"]).to(DEV), out_dtype=torch.bfloat16)
    got = y.cpu().view(torch.int16).numpy().view(np.uint16)
    fin = d["finite"]
    assert np.array_equal(got[:, fin], d["y_bits"][:, fin])
    assert torch.isnan(y.cpu()[:, ~torch.from_numpy(fin)].float()).all()


@pytest.mark.parametrize("N,K,seed", [(1024, 1024, 0), (1536, 7168, 1), (18432, 7168, 2), (7168, 18432, 3),
                                      (7168, 2048, 4), (2048, 7168, 5), (200, 300, 6), (1, 128, 7), (130, 1000, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_weight_dequant_bit_exact(N, K, seed, dtype):
    if dtype == torch.float32 and N * K > 20_000_000:
        pytest.skip("fp32 flavour is covered at the smaller shapes")
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x3A
    s = torch.rand((N + 127) // 128, (K + 127) // 128, generator=g) * 3e-3 + 1e-5
    ref = O.weight_dequant(codes.view(FP8), s, dtype=dtype)
    got = m.weight_dequant(codes.view(FP8).to(DEV), s.to(DEV), out_dtype=dtype)
    assert got.dtype == dtype and got.shape == (N, K)
    assert torch.equal(got.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))


def test_weight_dequant_honours_default_dtype():
    codes = torch.randint(0, 120, (128, 256), dtype=torch.uint8).view(FP8).to(DEV)
    s = torch.ones(1, 2, device=DEV)
    old = torch.get_default_dtype()
    try:
        torch.set_default_dtype(torch.bfloat16)
        assert m.weight_dequant(codes, s).dtype == torch.bfloat16
    finally:
        torch.set_default_dtype(old)
    assert m.weight_dequant(codes, s).dtype == torch.float32


def test_quantize_then_dequantize_round_trip_bound():
    """Size-independent property at the full C3 weight shape: |dequant(quant(w)) - w| <= half an
    e4m3 ulp of the block maximum's grid, i.e. <= s * 16 (= 2**4, half of the top binade's step 32)."""
    w, _, _ = P.weights(2048, 7168, 10)
    wd = w.to(DEV)
    q, s, _, _ = m.quant_weight(wd, True)
    back = m.weight_dequant(q, s, out_dtype=torch.float32)
    sfull = s.repeat_interleave(128, 0).repeat_interleave(128, 1)
    assert torch.all((back - wd.float()).abs() <= sfull * 16.0 * (1 + 1e-6))


# ------------------------------------------------------------------ add_bias
@pytest.mark.parametrize("M,N", [(128, 1024), (5, 18432), (7, 100), (1, 7)])
def test_add_bias_bit_exact(M, N):
    g = torch.Generator().manual_seed(M * 31 + N)
    x = torch.randn(M, N, generator=g).bfloat16()
    b = torch.randn(N, generator=g).bfloat16()
    ref = O.add_bias(x, b)
    xd = x.to(DEV)
    out = m.add_bias(xd, b.to(DEV))
    assert out.data_ptr() == xd.data_ptr()
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


# ------------------------------------------------------------------ random ragged shapes, every quantizer
def test_quantizers_random_shapes():
    """40 seeded shapes with ragged sides (and, for every fourth, a strided view as the input): every
    quantizer against the oracle, bytes, scales, shapes and strides."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        M = int(rng.choice([1, 3, 8, 63, 64, 65, 129, 257, 520])) + int(rng.integers(0, 5))
        K = int(rng.choice([1, 7, 128, 130, 511, 512, 640, 1100])) + int(rng.integers(0, 9))
        kind = ("normal", "outliers", "heavy")[case % 3]
        x = P.activations(kind, M, K + 16, case)
        if case % 5 == 0:
            x[0, 8] = 3e4                                   # saturates the DeepLinear dialect
        xd = x.to(DEV)
        if case % 4 == 0:                                   # row stride K + 16, 16-byte offset
            x, xd = x[:, 8:8 + K], xd[:, 8:8 + K]
        else:
            x, xd = x[:, :K].contiguous(), xd[:, :K].contiguous()
        tag = (case, M, K)
        if K % 128 == 0:                                    # the official quantizer wants whole groups
            y, s = m.act_quant(xd)
            yr, sr = O.act_quant(x.contiguous())
            assert np.array_equal(u8(y), u8(yr)) and torch.equal(s.cpu(), sr), tag
        _same_quant([t for t in m.quant_input(xd, True) if t is not None],
                    [t for t in O.quant_input(x, True) if t is not None])
        _same_quant(m.quant_input(xd, False), O.quant_input(x, False))
        _same_quant(m.quant_grad_output(xd), O.quant_grad_output(x))
        for only_forward in (True, False):
            _same_quant([t for t in m.quant_weight(xd, only_forward) if t is not None],
                        [t for t in O.quant_weight(x, only_forward) if t is not None])


def test_quant_input_broadcast_rows():
    """A row expanded to M rows (row stride 0) is quantized like its materialised copy, as the training quantizer
    already does; the C entry point still rejects overlapping rows of any other stride."""
    g = torch.Generator().manual_seed(12)
    row = torch.randn(1, 512, generator=g).bfloat16()
    x = row.to(DEV).expand(12, 512)
    assert x.stride(0) == 0
    y, s, _, _ = m.quant_input(x, True)
    yr, sr, _, _ = O.quant_input(row.expand(12, 512).contiguous(), True)
    assert torch.equal(y.cpu().view(torch.uint8), yr.view(torch.uint8)) and torch.equal(s.cpu().contiguous(), sr.contiguous())
    from mdy_triton_amd import _lib
    L = _lib.load()
    buf = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    p = buf.data_ptr()
    assert L.mdy_act_quant(p, p + 1024, p + 2048, 4, 128, 64, 4, 128, 1, 1, 0, None) == -2
    assert L.mdy_act_quant(p, p + 1024, p + 2048, 1, 128, 64, 1, 128, 1, 1, 0, None) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("xd,yd", [(torch.float32, torch.bfloat16), (torch.float32, torch.float32),
                                   (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_add_grad_bit_exact(xd, yd):
    """main_grad += wgrad (megatron_patchs/add_kernel.py:55-62): one fp32 add and one rounding, so bit-exact against the
    oracle (and against numpy's float32 add for the fp32 accumulator); odd sizes take the masked tail."""
    from mdy_triton_amd.megatron_patchs.add_kernel import add_grad
    from mdy_triton_amd.megatron_patchs.manger import CustomManger
    g = torch.Generator().manual_seed(3)
    for shape in ((1,), (2047,), (300, 513), (4, 128, 256)):
        x = torch.randn(*shape, generator=g).to(xd)
        y = (torch.randn(*shape, generator=g) * 3).to(yd)
        want = O.add_grad(x, y)
        xg = x.to(DEV)
        out = CustomManger.add_grad(xg, y.to(DEV))
        assert out.data_ptr() == xg.data_ptr() and out.dtype == xd
        assert torch.equal(out.cpu().view(torch.int32 if xd == torch.float32 else torch.int16),
                           want.view(torch.int32 if xd == torch.float32 else torch.int16))
        if xd == torch.float32:
            assert np.array_equal(out.cpu().numpy(), x.numpy() + y.float().numpy())
    with pytest.raises(AssertionError):
        add_grad(torch.zeros(4, 4, device=DEV).t(), torch.zeros(4, 4, device=DEV))
    with pytest.raises(TypeError):
        add_grad(torch.zeros(4, device=DEV, dtype=torch.float16), torch.zeros(4, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(128, 1024), (37, 384), (1, 7168), (300, 2048)])
def test_act_quant_and_quant_input_fp16_fp32_inputs(dtype, M, K):
    """The reference kernels load with .to(tl.float32), so fp16 and fp32 tensors are quantized from their exact
    fp32 values (offical_kernel.py:12, fp8.py:108): bytes and scales bit-exact against the oracle, whose arithmetic
    is dtype-agnostic.  fp32 values are not bf16-representable in general, so this also exercises group maxima and
    quotients that the bf16 kernel never sees."""
    g = torch.Generator().manual_seed(M + K)
    x = (torch.randn(M, K, generator=g) * torch.rand(M, 1, generator=g) * 8).to(dtype)
    x[0, :3] = torch.tensor([0.0, -0.0, 1e-6]).to(dtype)
    y_ref, s_ref = O.act_quant(x)
    y, s = m.act_quant(x.to(DEV))
    assert y.dtype == FP8 and y.shape == x.shape and s.shape == (M, K // 128)
    assert torch.equal(y.cpu().view(torch.uint8), y_ref.view(torch.uint8)) and torch.equal(s.cpu(), s_ref)
    q, qs, _, _ = m.quant_input(x.to(DEV), True)
    rq, rqs, _, _ = O.quant_input(x, True)
    assert torch.equal(q.cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(qs.cpu().contiguous(), rqs.contiguous())
    # a row-strided view (column slice of a wider tensor) takes the element-wise loads
    wide = torch.randn(M, K + 24, generator=g).to(dtype)
    q2, qs2, _, _ = m.quant_input(wide.to(DEV)[:, 8:8 + K], True)
    rq2, rqs2, _, _ = O.quant_input(wide[:, 8:8 + K], True)
    assert torch.equal(q2.cpu().view(torch.uint8), rq2.view(torch.uint8)) and torch.equal(qs2.cpu().contiguous(), rqs2.contiguous())
    with pytest.raises(TypeError):
        m.act_quant(torch.zeros(4, 128, device=DEV, dtype=torch.float64))


@pytest.mark.parametrize("bs", [8, 32, 64, 256, 512])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_act_quant_and_weight_dequant_other_block_sizes(bs, dtype):
    """act_quant(x, block_size) and weight_dequant(x, s, block_size) take any block size in the reference
    (offical_kernel.py:21-27, 46-53); here every power of two from 8 (to 512 for the quantizer): bit-exact
    against the oracle, including a ragged weight whose edge blocks are partial."""
    g = torch.Generator().manual_seed(bs)
    M, K = 37, 1024
    x = (torch.randn(M, K, generator=g) * torch.rand(M, 1, generator=g) * 4).to(dtype)
    y_ref, s_ref = O.act_quant(x, bs)
    y, s = m.act_quant(x.to(DEV), bs)
    assert s.shape == (M, K // bs)
    assert torch.equal(y.cpu().view(torch.uint8), y_ref.view(torch.uint8)) and torch.equal(s.cpu(), s_ref)
    N2, K2 = 300, 776
    wq = torch.randint(0, 0x7F, (N2, K2), generator=g, dtype=torch.uint8).view(FP8)
    ws = torch.rand((N2 + bs - 1) // bs, (K2 + bs - 1) // bs, generator=g) + 0.25
    for od in (torch.bfloat16, torch.float32):
        got = m.weight_dequant(wq.to(DEV), ws.to(DEV), bs, out_dtype=od)
        ref = O.weight_dequant(wq, ws, bs, dtype=od)
        assert torch.equal(got.cpu().view(torch.int16 if od == torch.bfloat16 else torch.int32),
                           ref.view(torch.int16 if od == torch.bfloat16 else torch.int32))
    with pytest.raises(ValueError):
        m.act_quant(x.to(DEV)[:, :960].contiguous(), 96)
    with pytest.raises(ValueError):
        m.weight_dequant(wq.to(DEV), ws.to(DEV), 100)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_and_training_quantizers_fp16_fp32_inputs(dtype):
    """Every quantizer takes fp16 and fp32 tensors like the reference's kernels (.to(tl.float32) on load): the block
    weight quantizers (an fp32 master weight), the training quantizers with their transposed copies, and the
    official-dialect pair; all bit-exact against the oracle, whose arithmetic is dtype-agnostic."""
    g = torch.Generator().manual_seed(17)
    w = (torch.randn(300, 520, generator=g) * 0.02).to(dtype)
    for only_forward in (True, False):
        got = m.quant_weight(w.to(DEV), only_forward)
        ref = O.quant_weight(w, only_forward)
        for a, b in zip(got, ref):
            assert (a is None) == (b is None)
            if a is not None:
                assert torch.equal(a.cpu().contiguous().view(torch.uint8) if a.dtype == FP8 else a.cpu(), b.contiguous().view(torch.uint8) if b.dtype == FP8 else b)
    wb = (torch.randn(256, 384, generator=g) * 0.02).to(dtype)
    y, s = m.weight_quant_block(wb.to(DEV), dtype=FP8)
    yr, sr = O.weight_quant_block(wb)
    assert torch.equal(y.cpu().view(torch.uint8), yr.view(torch.uint8)) and torch.equal(s.cpu(), sr)
    yt, st = m.weight_quant_block(wb.to(DEV).t(), dtype=FP8)                   # strided (transposed view)
    ytr, str_ = O.weight_quant_block(wb.t().contiguous())
    assert torch.equal(yt.cpu().view(torch.uint8), ytr.view(torch.uint8)) and torch.equal(st.cpu(), str_)
    x = torch.randn(300, 512, generator=g).to(dtype)
    for fn, ofn in ((lambda t: m.quant_input(t, False), lambda t: O.quant_input(t, False)), (m.quant_grad_output, O.quant_grad_output),
                    (lambda t: m.per_token_cast_to_fp8(t, True), lambda t: O.per_token_cast_to_fp8(t, True))):
        for a, b in zip(fn(x.to(DEV)), ofn(x)):
            a, b = a.cpu().contiguous(), b.contiguous()
            assert a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype == FP8 else a, b.view(torch.uint8) if b.dtype == FP8 else b)
    yb, sb = m.act_quant_block(x.to(DEV), transpose=True, dtype=FP8)
    ybr, sbr = O.act_quant_block(x, transpose=True)
    assert torch.equal(yb.cpu().view(torch.uint8), ybr.view(torch.uint8)) and torch.equal(sb.cpu(), sbr)
    q = m.per_block_cast_to_fp8([w.to(DEV), (w * 2).to(DEV)], output_transpose=True)
    qr = O.per_block_cast_to_fp8([w, w * 2], output_transpose=True)
    for a, b in zip(q, qr):
        assert torch.equal(a.cpu().view(torch.uint8) if a.dtype == FP8 else a.cpu(), b.view(torch.uint8) if b.dtype == FP8 else b)


def test_deep_linear_and_fp8_linear_with_fp32_parameters():
    """nn.Linear's default dtype: fp32 weight, bias and input.  The forward quantizes them from their exact values and
    returns bf16 like the reference's GEMM; the bias is added in fp32."""
    g = torch.Generator().manual_seed(23)
    x = torch.randn(64, 512, generator=g)
    with torch.no_grad():
        lin = m.DeepLinear(512, 256, bias=True)
        assert lin.weight.dtype == torch.float32
        lin.weight.copy_(torch.randn(256, 512, generator=g) * 0.03)
        lin.bias.copy_(torch.randn(256, generator=g))
        ref = O.deep_linear_forward(x, lin.weight.detach(), None).float() + lin.bias.detach()
        lin = lin.to(DEV)
        out = lin(x.to(DEV))
        lin.fuse_bias = True                       # not fusable with an fp32 bias: falls back to the separate add
        assert torch.equal(lin(x.to(DEV)), out)
    assert out.dtype == torch.bfloat16
    mag = torch.maximum(ref.abs(), (ref - lin.bias.detach().cpu()).abs())
    assert bool(((out.float().cpu() - ref).abs() <= 2e-2 + 1e-2 * mag).all())
    nb = torch.randn(8, 200, generator=g).bfloat16()
    bias = torch.randn(200, generator=g)
    got = m.add_bias(nb.clone().to(DEV), bias.to(DEV))
    assert torch.equal(got.cpu(), (nb.float() + bias).bfloat16())
    with torch.no_grad():
        fl = m.Fp8Linear(512, 256, bias=True, fp8_dtype=FP8)
        fl.weight.copy_(lin.weight.cpu()); fl.bias.copy_(lin.bias.cpu())
        ref2 = O.fp8_linear_forward(x, fl.weight.detach(), None).float() + fl.bias.detach()
        out2 = fl.to(DEV)(x.to(DEV))
    assert bool(((out2.float().cpu() - ref2).abs() <= 2e-2 + 1e-2 * mag).all())
