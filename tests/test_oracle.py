"""Pins the CPU oracle (oracle/oracle.py) from outside its own formulas: golden
fixtures derived from the format definition, numpy re-derivations, invariants,
float64 truth and exactly-representable GEMM cases."""
import os

import numpy as np
import pytest
import torch

from oracle import fp8_format as F
from oracle import oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")
FP8 = torch.float8_e4m3fn


def bf16_from_bits(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.astype(np.uint16).view(np.int16).copy()).view(torch.bfloat16)


def u8(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy()


# ------------------------------------------------------------------ act_quant
def test_act_quant_golden_codes():
    d = np.load(os.path.join(GOLD, "act_quant_codes.npz"))
    x = bf16_from_bits(d["x_bits"])
    y, s = O.act_quant(x)
    assert np.array_equal(u8(y), d["y"])
    assert np.array_equal(s.numpy().view(np.uint32), d["s"].view(np.uint32))


def test_act_quant_numpy_rederivation_and_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 1024, generator=g).bfloat16()
    x[3, 5] *= 50  # an outlier group
    y, s = O.act_quant(x)
    xf = F.bf16_bits_to_f32(x.view(torch.int16).numpy().view(np.uint16)).reshape(-1, 128)
    amax = np.abs(xf).max(axis=1)
    s_np = (amax / np.float32(448.0)).astype(np.float32)
    assert np.array_equal(s.numpy().reshape(-1).view(np.uint32), s_np.view(np.uint32))
    y_np = F.encode_rne((xf / s_np[:, None]).astype(np.float32))
    assert np.array_equal(u8(y).reshape(-1, 128), y_np)
    # the absmax element encodes to +-448
    assert np.all((y_np & 0x7F).max(axis=1) == 0x7E)
    # reconstruction error at most half an e4m3 ulp of the quotient (8 ulps of 2**-3 relative, or the subnormal step)
    q = xf / s_np[:, None]
    deq = F.decode(y_np)
    ulp = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(q), 2.0 ** -6))) - 3), 2.0 ** -9)
    assert np.all(np.abs(deq - q) <= ulp / 2 * (1 + 1e-6))


def test_act_quant_idempotent_on_its_own_output():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(16, 256, generator=g).bfloat16()
    y, s = O.act_quant(x)
    # use power-of-two scales so that the dequantized tensor is exact in bf16
    s2 = torch.exp2(torch.floor(torch.log2(s)))
    xd = (y.float().reshape(16, 2, 128) * s2[:, :, None]).reshape(16, 256)
    y[:, 0] = torch.tensor(448.0).to(FP8)  # make sure the absmax is 448 in group 0 of every row
    y[:, 128] = torch.tensor(-448.0).to(FP8)
    xd = (y.float().reshape(16, 2, 128) * s2[:, :, None]).reshape(16, 256).bfloat16()
    y2, s3 = O.act_quant(xd)
    assert torch.equal(s3, s2)
    assert np.array_equal(u8(y2), u8(y))


def test_act_quant_zero_group_is_nan_and_negative_zero_keeps_sign():
    x = torch.zeros(1, 256, dtype=torch.bfloat16)
    x[0, 128] = 1.0
    x[0, 129] = -0.0
    y, s = O.act_quant(x)
    b = u8(y)[0]
    assert s[0, 0] == 0 and np.all((b[:128] & 0x7F) == 0x7F)
    assert b[128] == 0x7E and b[129] == 0x80 and b[130] == 0x00


# ------------------------------------------------------------------ weight_dequant
def test_weight_dequant_golden_codes():
    d = np.load(os.path.join(GOLD, "weight_dequant_codes.npz"))
    x = torch.from_numpy(d["x"]).view(FP8)
    y = O.weight_dequant(x, torch.from_numpy(d["s"]), dtype=torch.bfloat16)
    got = y.view(torch.int16).numpy().view(np.uint16)
    fin = d["finite"]
    assert np.array_equal(got[:, fin], d["y_bits"][:, fin])
    assert torch.isnan(y[:, ~torch.from_numpy(fin)].float()).all()


def test_weight_dequant_numpy_rederivation_ragged():
    rng = np.random.default_rng(5)
    N, K = 200, 300
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x3C
    s = rng.uniform(1e-4, 3e-3, size=(2, 3)).astype(np.float32)
    y = O.weight_dequant(torch.from_numpy(codes).view(FP8), torch.from_numpy(s), dtype=torch.bfloat16)
    sfull = np.repeat(np.repeat(s, 128, 0)[:N], 128, 1)[:, :K]
    prod = (F.decode(codes) * sfull).astype(np.float32)
    assert np.array_equal(y.view(torch.int16).numpy().view(np.uint16), F.f32_to_bf16_bits_rne(prod))
    y32 = O.weight_dequant(torch.from_numpy(codes).view(FP8), torch.from_numpy(s), dtype=torch.float32)
    assert np.array_equal(y32.numpy().view(np.uint32), prod.view(np.uint32))


# ------------------------------------------------------------------ fp8_gemm
def _rand_problem(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    a, a_s = O.act_quant(x)
    Np = (N + 127) // 128 * 128
    wp = torch.zeros(Np, K, dtype=torch.bfloat16)
    wp[:N] = w
    wp[N:] = 0.01
    b, b_s = O.weight_quant_block(wp)
    return x, w, a, a_s, b[:N].contiguous(), b_s


def test_fp8_gemm_golden_exact():
    d = np.load(os.path.join(GOLD, "gemm_exact.npz"))
    a = torch.from_numpy(d["a"]).view(FP8)
    b = torch.from_numpy(d["b"]).view(FP8)
    a_s, b_s = torch.from_numpy(d["a_s"]), torch.from_numpy(d["b_s"])
    for fn in (O.fp8_gemm, O.fp8_gemm_blockwise):
        c32 = fn(a, a_s, b, b_s, dtype=torch.float32)
        assert np.array_equal(c32.numpy().view(np.uint32), d["c_f32"].view(np.uint32))
        c16 = fn(a, a_s, b, b_s, dtype=torch.bfloat16)
        assert np.array_equal(c16.view(torch.int16).numpy().view(np.uint16), d["c_bf16_bits"])
    assert np.array_equal(O.fp8_gemm_f64(a, a_s, b, b_s).numpy(), d["c_f32"].astype(np.float64))


def test_fp8_gemm_against_float64_and_blockwise():
    x, w, a, a_s, b, b_s = _rand_problem(48, 200, 512, 11)
    truth = O.fp8_gemm_f64(a, a_s, b, b_s)
    c = O.fp8_gemm(a, a_s, b, b_s, dtype=torch.float32).double()
    cb = O.fp8_gemm_blockwise(a, a_s, b, b_s, dtype=torch.float32).double()
    scale = truth.abs().max()
    assert (c - truth).abs().max() <= 1e-5 * scale
    assert (cb - truth).abs().max() <= 1e-5 * scale
    # and it approximates the unquantized product at the level the reference reports
    ref = x.float() @ w.float().t()
    assert (c.float() - ref).abs().mean() < 0.05 * ref.abs().mean() + 1e-3


def test_fp8_gemm_one_hot_rows_and_single_scale_block():
    N, K = 256, 256
    g = torch.Generator().manual_seed(2)
    b = torch.randint(0, 0x77, (N, K), generator=g, dtype=torch.uint8).view(FP8)
    b_s = torch.tensor([[1.0, 0.5], [0.25, 2.0]])
    a = torch.zeros(4, K).to(FP8)
    hot = [3, 127, 128, 255]
    for r, k in enumerate(hot):
        a[r, k] = torch.tensor(1.0).to(FP8)
    a_s = torch.tensor([[1.0, 1.0], [2.0, 1.0], [1.0, 4.0], [1.0, 0.5]])
    c = O.fp8_gemm(a, a_s, b, b_s, dtype=torch.float32)
    bd = O.weight_dequant(b, b_s, dtype=torch.float32)
    for r, k in enumerate(hot):
        assert torch.equal(c[r], bd[:, k] * a_s[r, k // 128])
    # perturbing one (n-block, k-block) weight scale changes only that output stripe
    b_s2 = b_s.clone()
    b_s2[1, 0] = 8.0
    a2 = torch.randint(0, 0x60, (8, K), generator=g, dtype=torch.uint8).view(FP8)
    a2_s = torch.ones(8, 2)
    d = O.fp8_gemm(a2, a2_s, b, b_s2, dtype=torch.float32) - O.fp8_gemm(a2, a2_s, b, b_s, dtype=torch.float32)
    assert torch.count_nonzero(d[:, :128]) == 0 and torch.count_nonzero(d[:, 128:]) > 0


# ------------------------------------------------------------------ DeepLinear dialect
def test_quant_input_layout_padding_and_eps():
    g = torch.Generator().manual_seed(4)
    M, K = 6, 300
    x = torch.randn(M, K, generator=g).bfloat16()
    y, s, y_t, s_t = O.quant_input(x, True)
    assert y_t is None and s_t is None
    assert tuple(y.shape) == (8, 512) and tuple(s.shape) == (8, 4) and s.stride() == (1, 8)
    yb = u8(y)
    assert np.all(yb[M:] == 0) and np.all(yb[:, 384:] == 0) and np.all(yb[:M, K:384] == 0)
    eps_scale = (np.float32(1e-8) / np.float32(448)).astype(np.float32)
    assert np.all(s.numpy()[M:] == eps_scale) and np.all(s.numpy()[:, 3] == eps_scale)
    xf = x.float().numpy()
    amax = np.abs(xf[:, :128]).max(axis=1)
    s_np = ((np.minimum(amax, np.float32(1e4)) + np.float32(1e-8)) / np.float32(448)).astype(np.float32)
    assert np.array_equal(s.numpy()[:M, 0].view(np.uint32), s_np.view(np.uint32))
    assert np.array_equal(yb[:M, :128], F.encode_rne_sat((xf[:, :128] / s_np[:, None]).astype(np.float32)))


def test_quant_input_saturates_beyond_clamp():
    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    x[0, 0] = 3e4
    x[0, 1] = -2e4
    x[0, 2] = 5e3
    y, s, _, _ = O.quant_input(x, True)
    b = u8(y)[0]
    assert b[0] == 0x7E and b[1] == 0xFE
    sc = (np.float32(1e4) + np.float32(1e-8)) / np.float32(448)
    assert s[0, 0].item() == sc
    assert b[2] == F.encode_rne(np.array([np.float32(5e3) / sc], np.float32))[0]


def test_quant_weight_blocks_padding_transpose():
    g = torch.Generator().manual_seed(6)
    N, K = 200, 300
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    y, s, y_t, s_t = O.quant_weight(w, False)
    assert tuple(y.shape) == (256, 512) and tuple(s.shape) == (2, 4)
    assert tuple(y_t.shape) == (512, 256) and tuple(s_t.shape) == (4, 2)
    assert torch.equal(y_t.view(torch.uint8), y.view(torch.uint8).t()) and torch.equal(s_t, s.t())
    y1, s1, _, _ = O.quant_weight(w, True)
    assert tuple(y1.shape) == (256, 512)
    wf = w.float().numpy()
    blk = wf[128:200, 256:300]
    amax = np.abs(blk).max()
    sc = ((np.float32(amax) + np.float32(1e-8)) / np.float32(448)).astype(np.float32)
    assert s1[1, 2].item() == sc
    assert sc != np.float32(amax) / np.float32(448)  # the eps is not a no-op at this magnitude
    assert np.array_equal(u8(y1)[128:200, 256:300], F.encode_rne_sat((blk / sc).astype(np.float32)))
    assert np.all(u8(y1)[200:] == 0)


def test_weight_quant_block_matches_act_quant_on_uniform_rows():
    # a 128x128 block whose rows all share the same absmax quantizes like 128 act_quant groups
    g = torch.Generator().manual_seed(8)
    w = torch.randn(128, 128, generator=g).bfloat16()
    w[:, 0] = 7.0
    w = w.clamp(-7, 7)
    yb, sb = O.weight_quant_block(w)
    ya, sa = O.act_quant(w)
    assert torch.equal(sa, sb.expand(128, 1)) and np.array_equal(u8(ya), u8(yb))


def test_quant_grad_output_is_row_and_column_quant():
    g = torch.Generator().manual_seed(9)
    dy = torch.randn(256, 256, generator=g).bfloat16()
    y, s, y_t, s_t = O.quant_grad_output(dy)
    y_r, s_r, _, _ = O.quant_input(dy, True)
    assert np.array_equal(u8(y), u8(y_r)) and torch.equal(s.contiguous(), s_r.contiguous())
    y_c, s_c, _, _ = O.quant_input(dy.t().contiguous(), True)
    assert np.array_equal(u8(y_t), u8(y_c)) and torch.equal(s_t.contiguous(), s_c.contiguous())


def test_add_bias_and_deep_linear_composition():
    g = torch.Generator().manual_seed(10)
    x = torch.randn(2, 4, 256, generator=g).bfloat16()
    w = (torch.randn(128, 256, generator=g) * 0.05).bfloat16()
    bias = torch.randn(128, generator=g).bfloat16()
    out = O.deep_linear_forward(x, w, bias)
    assert tuple(out.shape) == (2, 4, 128) and out.dtype == torch.bfloat16
    ref = torch.nn.functional.linear(x.float(), w.float(), bias.float())
    assert (out.float() - ref).abs().mean() < 0.03
    nb = O.deep_linear_forward(x, w, None)
    assert torch.equal(out, O.add_bias(nb, bias))


def test_add_bias_numpy_pin():
    """add_bias (fp8.py:283-305) from outside the oracle: bf16 bits -> fp32, one fp32 add, round to nearest
    even back to bf16, all in numpy with the from-definition conversions.  Includes ties (a bias of half an
    ulp of x), cancellation to zero, a sum that overflows bf16 and a dropped-term check (a zero bias must be
    the identity)."""
    g = torch.Generator().manual_seed(21)
    x = torch.randn(37, 200, generator=g).bfloat16()
    b = torch.randn(200, generator=g).bfloat16()
    x[0, :4] = torch.tensor([1.0, 1.0, 256.0, 3.0e38]).bfloat16()
    b[:4] = torch.tensor([2.0 ** -8, -1.0, 1.0, 3.0e38]).bfloat16()       # tie to even, exact zero, tie, overflow
    xb = x.view(torch.int16).numpy().view(np.uint16)
    bb = b.view(torch.int16).numpy().view(np.uint16)
    want = F.f32_to_bf16_bits_rne(F.bf16_bits_to_f32(xb) + F.bf16_bits_to_f32(bb)[None, :])
    got = O.add_bias(x.clone(), b)
    assert got.dtype == torch.bfloat16 and got.shape == x.shape
    assert np.array_equal(got.view(torch.int16).numpy().view(np.uint16), want)
    assert got[0, 0].item() == 1.0 and got[0, 1].item() == 0.0 and np.isinf(got[0, 3].item())
    assert torch.equal(O.add_bias(x.clone(), torch.zeros(200).bfloat16()), x)
    # leading dimensions broadcast over the last one only
    x3 = x[:36].reshape(3, 12, 200)
    assert torch.equal(O.add_bias(x3.clone(), b).reshape(36, 200), got[:36])


def test_quant_input_training_outputs():
    # the transposed copy is a 128x128 block quantization: it must coincide with the block weight quantizer's
    g = torch.Generator().manual_seed(11)
    x = torch.randn(256, 512, generator=g).bfloat16()
    x[3, 5] = 2e4                                      # beyond the clamp: saturates in both
    y, s, y_t, s_t = O.quant_input(x, False)
    y1, s1, _, _ = O.quant_input(x, True)
    assert np.array_equal(u8(y), u8(y1)) and torch.equal(s.contiguous(), s1.contiguous())
    _, _, w_t, ws_t = O.quant_weight(x, False)
    assert tuple(y_t.shape) == (512, 256) and tuple(s_t.shape) == (4, 2)
    assert np.array_equal(u8(y_t), u8(w_t)) and torch.equal(s_t, ws_t)
    # ragged: rows padded to 256, padding bytes 0, padded tiles carry the eps scale
    xr = torch.randn(130, 300, generator=g).bfloat16()
    y, s, y_t, s_t = O.quant_input(xr, False)
    assert tuple(y.shape) == (256, 512) and tuple(y_t.shape) == (512, 256) and tuple(s_t.shape) == (4, 2)
    assert np.all(u8(y_t)[300:] == 0) and np.all(u8(y_t)[:, 130:] == 0)
    assert s_t[3, 0].item() == np.float32(1e-8) / np.float32(448)
    # brute force of one tile: block (rows 128..129, cols 256..299)
    blk = xr.float().numpy()[128:130, 256:300]
    sc = ((np.abs(blk).max() + np.float32(1e-8)) / np.float32(448)).astype(np.float32)
    assert s_t[2, 1].item() == sc
    assert np.array_equal(u8(y_t)[256:300, 128:130], F.encode_rne_sat((blk / sc).astype(np.float32)).T)


def test_quant_grad_output_ragged_layout():
    g = torch.Generator().manual_seed(12)
    dy = torch.randn(130, 200, generator=g).bfloat16()
    y, s, y_t, s_t = O.quant_grad_output(dy)
    assert tuple(y.shape) == (256, 256) and tuple(s.shape) == (256, 2) and s.stride() == (1, 256)
    assert tuple(y_t.shape) == (256, 256) and tuple(s_t.shape) == (256, 2) and s_t.stride() == (1, 256)
    d = dy.float().numpy()
    # column 7, rows 128..129 form one group of the transposed copy
    col = d[128:130, 7]
    sc = ((np.abs(col).max() + np.float32(1e-8)) / np.float32(448)).astype(np.float32)
    assert s_t[7, 1].item() == sc
    assert np.array_equal(u8(y_t)[7, 128:130], F.encode_rne_sat((col / sc).astype(np.float32)))
    assert np.all(u8(y_t)[200:] == 0) and np.all(u8(y_t)[:, 130:] == 0)


def test_deep_linear_backward_close_to_unquantized_gradients():
    g = torch.Generator().manual_seed(13)
    x = torch.randn(2, 128, 256, generator=g).bfloat16()
    w = (torch.randn(256, 256, generator=g) * 0.05).bfloat16()
    dy = torch.randn(2, 128, 256, generator=g).bfloat16()
    dgrad, wgrad, gb = O.deep_linear_backward(x, w, dy)
    xf = x.float().reshape(-1, 256); dyf = dy.float().reshape(-1, 256)
    dref = (dyf @ w.float()).reshape(x.shape)
    wref = dyf.t() @ xf
    assert tuple(dgrad.shape) == tuple(x.shape) and tuple(wgrad.shape) == (256, 256)
    assert (dgrad.float() - dref).abs().mean() < 0.05 * dref.abs().mean()
    assert (wgrad.float() - wref).abs().mean() < 0.05 * wref.abs().mean()
    assert gb.dtype == torch.bfloat16 and torch.equal(gb, dyf.sum(0).bfloat16())
    # transposed operands really are transposes: swapping x and dy roles transposes wgrad
    _, wgrad2, _ = O.deep_linear_backward(dy.reshape(-1, 256), w, x.reshape(-1, 256))
    assert (wgrad2.float().t() - wref).abs().mean() < 0.05 * wref.abs().mean()


def test_silu_matches_torch_functional_and_autograd():
    g = torch.Generator().manual_seed(14)
    x = (torch.randn(16, 512, generator=g) * 2).bfloat16()
    for order in ("up-gate", "gate-up"):
        up, gate = (x[:, :256], x[:, 256:]) if order == "up-gate" else (x[:, 256:], x[:, :256])
        ref = (torch.nn.functional.silu(gate.float()) * up.float())
        act = O.silu_fwd(x, order)
        assert act.dtype == torch.bfloat16 and (act.float() - ref).abs().max() <= 2.0 ** -8 * ref.abs().max()
        xf = x.float().requires_grad_(True)
        upf, gatef = (xf[:, :256], xf[:, 256:]) if order == "up-gate" else (xf[:, 256:], xf[:, :256])
        dy = torch.randn(16, 256, generator=g).bfloat16()
        (torch.nn.functional.silu(gatef) * upf).backward(dy.float())
        dx = O.silu_bwd(dy, x, order)
        assert (dx.float() - xf.grad).abs().max() <= 2.0 ** -7 * xf.grad.abs().max()
    y, s, act = O.silu_act_quant(x)
    y2, s2 = O.act_quant(act)
    assert torch.equal(s, s2) and np.array_equal(u8(y), u8(y2))
    # closed forms: silu(0) = 0, silu(large) = identity, silu(-large) = -large * exp(-large)
    e = torch.tensor([[1.0, 1.0, 1.0, 0.0, 60.0, -60.0]]).bfloat16()
    got = O.silu_fwd(e).tolist()[0]
    assert got[:2] == [0.0, 60.0] and abs(got[2] / (-60.0 * np.exp(-60.0)) - 1) < 2.0 ** -8


def test_grouped_oracle_functions_reduce_to_the_pinned_ones():
    g = torch.Generator().manual_seed(15)
    x = torch.randn(512, 256, generator=g).bfloat16()
    # M % 256 == 0: per_token_cast_to_fp8(output_transpose) is quant_grad_output
    for a_, b_ in zip(O.per_token_cast_to_fp8(x, True), O.quant_grad_output(x)):
        assert a_.shape == b_.shape and a_.stride() == b_.stride()
        assert np.array_equal(u8(a_), u8(b_)) if a_.dtype == FP8 else torch.equal(a_.contiguous(), b_.contiguous())
    # rows pad to 128, not 256
    y, s, y_t, s_t = O.per_token_cast_to_fp8(x[:130], True)
    assert tuple(y.shape) == (256, 256) and tuple(y_t.shape) == (256, 256) and tuple(s_t.shape) == (256, 2)
    y, s, y_t, s_t = O.per_token_cast_to_fp8(x[:100], True)
    assert tuple(y.shape) == (128, 256) and tuple(s_t.shape) == (256, 1) and s.stride() == (1, 128)
    # grouped quantizer = the row quantizer on all rows + the transposed quantizer per group
    ya, sa, yts, sts = O.group_per_token_cast_to_fp8(x, [256, 256])
    yr, sr, _, _ = O.quant_input(x, True)
    assert np.array_equal(u8(ya), u8(yr)) and torch.equal(sa.contiguous(), sr.contiguous()) and sa.stride() == (1, 512)
    assert np.array_equal(u8(yts[1]), u8(O.quant_grad_output(x[256:])[2]))
    # block quantizer on a list = quant_weight per member
    ws = [(torch.randn(200, 300, generator=g) * 0.02).bfloat16() for _ in range(2)]
    yb, sb, ybt, sbt = O.per_block_cast_to_fp8(ws, True, True)
    q = O.quant_weight(ws[1], False)
    assert np.array_equal(u8(yb[1]), u8(q[0])) and torch.equal(sb[1], q[1]) and np.array_equal(u8(ybt[1]), u8(q[2])) and torch.equal(sbt[1], q[3])
    # grouped GEMM: rows of group g see only weight g
    qa, sa, _, _ = O.per_token_cast_to_fp8(x)
    qb, sb2 = O.per_block_cast_to_fp8([w[:128, :256].contiguous() for w in ws])
    out = O.fp8_grouped_matmul(qa, sa, qb, sb2, [300, 212])
    assert torch.equal(out[:300], O.fp8_gemm(qa[:300], sa.contiguous()[:300], qb[0], sb2[0]))
    assert torch.equal(out[300:], O.fp8_gemm(qa[300:], sa.contiguous()[300:], qb[1], sb2[1]))


def test_fp8_padding_row_by_row():
    """The padding pair against plain Python loops over rows (what the layout means, no tensor ops): every
    source row lands at slot_start[g] + r, every other destination row is zero, and unpadding is the inverse."""
    g = torch.Generator().manual_seed(31)
    m_splits = [3, 0, 256, 257, 1, 511]
    H = 5
    x = torch.randn(sum(m_splits), H, generator=g).bfloat16()
    padded, pads = O.fp8_padding(x, m_splits)
    assert pads == [256, 0, 256, 512, 256, 512] and padded.shape == (sum(pads), H)
    want = [[0.0] * H for _ in range(sum(pads))]
    src = dst = 0
    for m, pm in zip(m_splits, pads):
        assert dst % 256 == 0
        for r in range(m):
            want[dst + r] = x[src + r].float().tolist()
        src += m
        dst += pm
    assert padded.float().tolist() == want
    back = O.fp8_unpadding(padded, m_splits)
    assert torch.equal(back, x)
    assert O.fp8_padding(x[:0], [0, 0])[0].shape == (0, H)


def test_act_quant_block_transposed_reduces_to_act_quant_and_groups():
    """act_quant_block(x, transpose=True) == act_quant of the transposed, zero-padded matrix (the pinned
    quantizer), plus a plain loop over the groups of two columns: scale = max|.| / 448 in numpy float32 and
    bytes through the from-definition codec."""
    g = torch.Generator().manual_seed(41)
    for (M, N) in ((256, 128), (200, 256), (5, 128)):
        x = torch.randn(M, N, generator=g).bfloat16()
        y, s = O.act_quant_block(x, transpose=True)
        assert y.shape == (N, M) and s.shape == (N, (M + 127) // 128)
        PM = (M + 127) // 128 * 128
        xt = torch.zeros(N, PM).bfloat16()
        xt[:, :M] = x.t()
        y2, s2 = O.act_quant(xt)
        assert np.array_equal(u8(y), u8(y2[:, :M].contiguous())) and torch.equal(s, s2)
        xf = x.float().numpy()
        for col in (0, N - 1):
            for gi in range((M + 127) // 128):
                grp = xf[gi * 128:(gi + 1) * 128, col]
                sc = np.float32(np.abs(grp).max()) / np.float32(448.0)
                assert s[col, gi].item() == sc
                want = F.encode_rne((grp / sc).astype(np.float32))
                assert np.array_equal(u8(y)[col, gi * 128:gi * 128 + len(grp)], want)
    yy, ss = O.act_quant_block(x.reshape(1, 5, 128))
    ya, sa = O.act_quant(x.reshape(1, 5, 128))
    assert np.array_equal(u8(yy), u8(ya)) and torch.equal(ss, sa)


def test_rowscaled_matmul_float64_exact_and_reduction():
    g = torch.Generator().manual_seed(42)
    M, N, K = 40, 256, 384
    a = torch.randint(0, 0x78, (M, K), generator=g, dtype=torch.uint8).view(O.FP8)
    b = torch.randint(0, 0x78, (N, K), generator=g, dtype=torch.uint8).view(O.FP8)
    sa = torch.rand(M, 3, generator=g) + 0.5
    sb = torch.rand(N, 3, generator=g) + 0.5
    got = O.fp8_matmul_official(a, b, sa, sb, None, False)
    truth = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(3):
        part = a[:, kb * 128:(kb + 1) * 128].double() @ b[:, kb * 128:(kb + 1) * 128].double().t()
        truth += part * sa[:, kb].double()[:, None] * sb[:, kb].double()[None, :]
    assert (got.double() - truth).abs().max() <= 2 ** -8 * truth.abs().max()
    # weight-row scales constant within each 128-row block: the block-scaled GEMM (pinned) gives the same result
    sb_blk = torch.rand(2, 3, generator=g) + 0.5
    sb_rows = sb_blk.repeat_interleave(128, 0)
    assert torch.equal(O.fp8_matmul_official(a, b, sa, sb_rows, None, False), O.fp8_gemm(a, sa, b, sb_blk))
    # exactly representable: small integers, power-of-two scales (transposed scale roles would show)
    ai = torch.randint(-3, 4, (M, K), generator=g)
    bi = torch.randint(-3, 4, (N, K), generator=g)
    ea = torch.randint(-2, 3, (M, 3), generator=g)
    eb = torch.randint(-2, 3, (N, 3), generator=g)
    exact = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(3):
        exact += (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()) * \
            torch.exp2((ea[:, kb][:, None] + eb[:, kb][None, :]).double())
    out = O.fp8_matmul_official(ai.float().to(O.FP8), bi.float().to(O.FP8), torch.exp2(ea.float()), torch.exp2(eb.float()), None, False)
    assert torch.equal(out.double(), exact.to(torch.bfloat16).double())


def test_fp8_linear_oracle_close_to_unquantized():
    g = torch.Generator().manual_seed(43)
    x = torch.randn(4, 64, 256, generator=g).bfloat16()
    w = (torch.randn(128, 256, generator=g) * 0.05).bfloat16()
    b = torch.randn(128, generator=g).bfloat16()
    dy = torch.randn(4, 64, 128, generator=g).bfloat16()
    y = O.fp8_linear_forward(x, w, b)
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    assert y.shape == ref.shape and (y.float() - ref).abs().mean() < 0.03
    dx, dw, db = O.fp8_linear_backward(x, w, dy)
    dxr = dy.float() @ w.float()
    dwr = dy.float().reshape(-1, 128).t() @ x.float().reshape(-1, 256)
    assert dx.shape == x.shape and (dx.float() - dxr).abs().mean() < 0.06 * dxr.abs().mean()
    assert dw.shape == w.shape and (dw.float() - dwr).abs().mean() < 0.06 * dwr.abs().mean()
    assert torch.allclose(db.float(), dy.float().reshape(-1, 128).sum(0), rtol=1e-2, atol=1e-1)


def test_act_quant_block_e5m2_golden_codes():
    """The closed-form e5m2 fixture (tests/golden/make_fixtures.py, no oracle call): quantizing x along its rows must
    return, for every column, exactly the e5m2 codes it was built from and the power-of-two scale."""
    d = np.load(os.path.join(GOLD, "act_quant_block_e5m2.npz"))
    x = torch.from_numpy(d["x_bits"].view(np.int16)).view(torch.bfloat16)
    y_t, s_t = O.act_quant_block(x, transpose=True, dtype=torch.float8_e5m2)
    assert np.array_equal(y_t.view(torch.uint8).numpy(), d["y_t"]) and np.array_equal(s_t.numpy(), d["s_t"])
    # the row-wise direction of the transposed matrix is the same quantization
    y, s = O.act_quant_block(x.t().contiguous(), dtype=torch.float8_e5m2)
    assert np.array_equal(y.view(torch.uint8).numpy(), d["y_t"]) and np.array_equal(s.numpy(), d["s_t"])
