"""GPU parity of the official-dialect linear layer (deepseekv3/fp8_kernel.py: act_quant_block, fp8_matmul, Fp8Linear)
against the CPU oracle: quantizer bytes and scales bit-exact, GEMMs within rtol = atol = 1e-2, exactly
representable cases bit for bit."""
import math

import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from mdy_triton_amd import fp8_kernel as FK
from oracle import oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
DEV = "cuda:0"


def u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def close(got, ref):
    return torch.allclose(got.float().cpu(), ref.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M,N", [(256, 128), (1024, 7168), (200, 256), (5, 128), (4096, 1536), (129, 384)])
def test_act_quant_block_both_directions_bit_exact(M, N):
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, N, generator=g).bfloat16()
    x[min(3, M - 1), 5] = 300.0                      # an outlier sets one row group's and one column group's scale
    y_ref, s_ref = O.act_quant_block(x)
    yt_ref, st_ref = O.act_quant_block(x, transpose=True)
    y, s = m.act_quant_block(x.to(DEV), dtype=FP8)
    yt, st = m.act_quant_block(x.to(DEV), transpose=True, dtype=FP8)
    assert y.shape == (M, N) and s.shape == (M, N // 128) and yt.shape == (N, M) and st.shape == (N, (M + 127) // 128)
    assert yt.is_contiguous() and st.is_contiguous()
    assert np.array_equal(u8(y), u8(y_ref)) and torch.equal(s.cpu(), s_ref)
    assert np.array_equal(u8(yt), u8(yt_ref)) and torch.equal(st.cpu(), st_ref)
    # one pass for both copies (what the backward uses) and a strided input (a column slice of a wider tensor)
    y2, s2, yt2, st2 = FK._act_quant_transposed(x.to(DEV), True, "test")
    assert np.array_equal(u8(y2[:M]), u8(y_ref)) and torch.equal(s2[:M].cpu(), s_ref)
    assert np.array_equal(u8(yt2[:, :M]), u8(yt_ref)) and torch.equal(st2.cpu(), st_ref)
    wide = torch.randn(M, N + 64, generator=g).bfloat16().to(DEV)
    yt3, st3 = m.act_quant_block(wide[:, 32:32 + N], transpose=True, dtype=FP8)
    yt3_ref, st3_ref = O.act_quant_block(wide[:, 32:32 + N].cpu(), transpose=True)
    assert np.array_equal(u8(yt3), u8(yt3_ref)) and torch.equal(st3.cpu(), st3_ref)


def test_act_quant_block_leading_dims_and_asserts():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 3, 64, 256, generator=g).bfloat16()
    y, s = m.act_quant_block(x.to(DEV), dtype=FP8)
    yr, sr = O.act_quant_block(x)
    assert y.shape == x.shape and s.shape == (2, 3, 64, 2) and np.array_equal(u8(y), u8(yr)) and torch.equal(s.cpu(), sr)
    yt, st = m.act_quant_block(x.to(DEV), transpose=True, dtype=FP8)
    ytr, str_ = O.act_quant_block(x, transpose=True)
    assert yt.shape == (256, 384) and np.array_equal(u8(yt), u8(ytr)) and torch.equal(st.cpu(), str_)
    with pytest.raises(AssertionError):
        m.act_quant_block(torch.zeros(4, 100, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        m.act_quant_block(x.to(DEV), dtype=torch.float16)


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (256, 384, 512), (130, 200, 384), (1000, 260, 1024), (64, 64, 2304),
                                   (2048, 3328, 256), (1990, 3300, 384)])        # the last two: 128x256 tiles of the scheduled body
def test_rowscaled_gemm_exact_integer(M, N, K):
    """Integer operands and power-of-two scales on both sides: every product and sum is exact, so the bf16 result must
    equal the float64 computation rounded once (catches swapped scale roles, K-block order, tile edges)."""
    g = torch.Generator().manual_seed(M + N + K)
    ai = torch.randint(-3, 4, (M, K), generator=g)
    bi = torch.randint(-3, 4, (N, K), generator=g)
    KB = K // 128
    ea = torch.randint(-2, 3, (M, KB), generator=g)
    eb = torch.randint(-2, 3, (N, KB), generator=g)
    exact = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(KB):
        exact += (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()) * \
            torch.exp2((ea[:, kb][:, None] + eb[:, kb][None, :]).double())
    got = FK.fp8_matmul(ai.float().to(FP8).to(DEV), bi.float().to(FP8).to(DEV), torch.exp2(ea.float()).to(DEV),
                        torch.exp2(eb.float()).to(DEV), have_w=False) if M % 128 == 0 else \
        FK._matmul_rowscaled(ai.float().to(FP8).to(DEV), torch.exp2(ea.float()).to(DEV), bi.float().to(FP8).to(DEV),
                             torch.exp2(eb.float()).to(DEV), M, N, K, torch.device(DEV))
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu().double(), exact.to(torch.bfloat16).double())


def test_rowscaled_gemm_random_and_ragged_k():
    g = torch.Generator().manual_seed(9)
    M, N, K = 256, 300, 1000                            # K not a multiple of 128: completed with zeros
    x = torch.randn(K, M, generator=g).bfloat16()      # tokens x features: the operands are quantized transposes
    w = torch.randn(K, N, generator=g).bfloat16()
    a, sa = O.act_quant_block(x, transpose=True)        # [M, K], [M, 8]
    b, sb = O.act_quant_block(w, transpose=True)
    ref = O.fp8_matmul_official(a, b, sa, sb, None, False)
    got = FK.fp8_matmul(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV), have_w=False)
    assert got.shape == (M, N) and close(got, ref)
    with pytest.raises(AssertionError):
        FK.fp8_matmul(a[:100].to(DEV), b.to(DEV), sa[:100].to(DEV), sb.to(DEV), have_w=False)
    # the C entry point rejects what it cannot address
    from mdy_triton_amd import _lib
    L = _lib.load()
    one = torch.zeros(64, dtype=torch.uint8, device=DEV)
    p = one.data_ptr()
    assert L.mdy_fp8_gemm_nt_rowscaled(p, p, 1, 1, p, p, 1, 1, p, 4, 4, 100, 0, 0, None) == -2
    assert L.mdy_fp8_gemm_nt_rowscaled(p + 1, p, 1, 1, p, p, 1, 1, p, 4, 4, 128, 0, 0, None) == -3
    assert L.mdy_fp8_gemm_nt_rowscaled(None, p, 1, 1, p, p, 1, 1, p, 4, 4, 128, 0, 0, None) == -1
    assert L.mdy_fp8_gemm_nt_rowscaled(p, p, -1, 1, p, p, 1, 1, p, 4, 4, 128, 0, 0, None) == -2
    assert L.mdy_fp8_gemm_nt_rowscaled(p, p, 1, 1, p, p, 1, 1, p, 4, 4, 128, 5, 0, None) == -4
    assert L.mdy_act_quant_transpose(p, 0, None, p, p, p, 4, 128, 128, 1, 128, 128, 0, None) == -1
    assert L.mdy_act_quant_transpose(p, 7, p, p, p, p, 4, 128, 128, 1, 128, 128, 0, None) == -4     # unknown x_dtype
    assert L.mdy_act_quant_transpose(p, 0, p, p, p, p, 4, 128, 128, 1, 128, 128, 1, None) == -4     # mode 1 is not built


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape,N", [((2, 128, 256), 256), ((512, 1024), 768), ((3, 50, 384), 128), ((1024, 7168), 1536)])
def test_fp8_linear_forward_backward(shape, N, bias):
    g = torch.Generator().manual_seed(sum(shape) + N)
    K = shape[-1]
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    b = torch.randn(N, generator=g).bfloat16() if bias else None
    x = torch.randn(*shape, generator=g).bfloat16()
    dy = torch.randn(*shape[:-1], N, generator=g).bfloat16()
    ref_out = O.fp8_linear_forward(x, w, b)
    ref_dx, ref_dw, ref_db = O.fp8_linear_backward(x, w, dy, bias)
    lin = m.Fp8Linear(K, N, bias=bias, dtype=torch.bfloat16, fp8_dtype=torch.float8_e4m3fn)
    with torch.no_grad():
        lin.weight.copy_(w)
        if bias:
            lin.bias.copy_(b)
    lin = lin.to(DEV)
    xg = x.to(DEV).requires_grad_(True)
    out = lin(xg)
    out.backward(dy.to(DEV))
    assert out.shape == (*shape[:-1], N) and out.dtype == torch.bfloat16
    if bias:      # the relative part of the tolerance belongs to the GEMM result before the bias
        mag = torch.maximum(ref_out.float().abs(), (ref_out.float() - b.float()).abs())
        assert bool(((out.float().cpu() - ref_out.float()).abs() <= 1e-2 + 1e-2 * mag).all())
    else:
        assert close(out, ref_out)
    assert xg.grad.shape == x.shape and close(xg.grad, ref_dx)
    assert lin.weight.grad.shape == (N, K) and close(lin.weight.grad, ref_dw)
    if bias:
        assert torch.allclose(lin.bias.grad.float().cpu(), ref_db.float(), rtol=1e-2, atol=1e-2)
    # only one of the two gradients wanted
    lin.zero_grad()
    lin(x.to(DEV)).backward(dy.to(DEV))
    assert close(lin.weight.grad, ref_dw)
    lin.weight.requires_grad_(False)
    xg2 = x.to(DEV).requires_grad_(True)
    lin(xg2).backward(dy.to(DEV))
    assert close(xg2.grad, ref_dx)
    with pytest.raises(TypeError, match="float8_e4m3fn"):
        m.Fp8Linear(K, N, dtype=torch.bfloat16, fp8_dtype=torch.bfloat16)


def test_fp8_linear_without_tokens():
    """An empty batch: empty output, zero weight gradient, empty input gradient (no kernel is given a zero extent)."""
    lin = m.Fp8Linear(256, 128, bias=True, dtype=torch.bfloat16, device=DEV, fp8_dtype=FP8)
    x = torch.zeros(0, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    out = lin(x)
    assert out.shape == (0, 128)
    out.sum().backward()
    assert x.grad.shape == (0, 256) and torch.count_nonzero(lin.weight.grad) == 0 and torch.count_nonzero(lin.bias.grad) == 0
    yt, st = m.act_quant_block(x.detach(), transpose=True, dtype=FP8)
    assert yt.shape == (256, 0) and st.shape == (256, 0)


def test_act_quant_block_non_finite_and_zero_groups():
    """The official dialect has no eps and no clamp (fp8_kernel.py:52-54): an all-zero group has scale 0 and NaN bytes
    (0 / 0), an infinite element makes its group's scale infinite (finite / inf = 0, inf / inf = NaN), and a NaN
    element is ignored by the group maximum (tl.max / v_max_f32) and stays NaN.  Both copies, compared with the oracle
    on the input whose NaNs are zeroed for the maximum only - the same convention as the forward quantizer's test."""
    g = torch.Generator().manual_seed(6)
    M, N = 256, 256
    x = torch.randn(M, N, generator=g).bfloat16()
    x[:128, 5] = 0.0                      # column group (0, 5) all zero
    x[7, 128:256] = 0.0                   # row group (7, 1) all zero
    x[200, 17] = float("inf")
    x[130, 140] = float("nan")
    y, s = m.act_quant_block(x.to(DEV), dtype=FP8)
    yt, st = m.act_quant_block(x.to(DEV), transpose=True, dtype=FP8)
    xz = torch.where(torch.isnan(x), torch.zeros_like(x), x)
    yr, sr = O.act_quant_block(xz)
    ytr, str_ = O.act_quant_block(xz, transpose=True)
    assert torch.equal(s.cpu(), sr) and torch.equal(st.cpu(), str_)
    assert s[7, 1].item() == 0.0 and st[5, 0].item() == 0.0 and math.isinf(s[200, 0].item()) and math.isinf(st[17, 1].item())
    def same(got, ref, nan_at):
        got = got.cpu().float()
        ref = ref.float().clone()
        ref[nan_at] = float("nan")
        return torch.equal(torch.isnan(got), torch.isnan(ref)) and torch.equal(got[~torch.isnan(ref)], ref[~torch.isnan(ref)])
    assert same(y, yr, (130, 140)) and same(yt, ytr, (140, 130))
    assert torch.isnan(y.cpu().float()[7, 128:256]).all() and torch.isnan(yt.cpu().float()[5, :128]).all()
    assert torch.isnan(y.cpu().float()[200, 17]) and (y.cpu().float()[200, :17] == 0).all()


def test_rowscaled_gemm_non_finite_values():
    """A NaN operand byte poisons exactly its output row / column; an infinite scale makes its row (or column) infinite
    with the sign of the block's partial sum, NaN where that sum is zero; a zero scale drops the block: the pattern of
    the reference's accumulation (fp8_kernel.py:196-203) evaluated block by block."""
    g = torch.Generator().manual_seed(13)
    M, N, K = 128, 200, 384
    a = torch.randint(-6, 7, (M, K), generator=g).float().to(FP8)
    b = torch.randint(-6, 7, (N, K), generator=g).float().to(FP8)
    sa = torch.rand(M, 3, generator=g) + 0.5
    sb = torch.rand(N, 3, generator=g) + 0.5
    a.view(torch.uint8)[1, 3] = 0x7F
    b.view(torch.uint8)[5, K - 1] = 0xFF
    sa[2, 2] = float("inf")
    sb[9, 0] = float("inf")
    sa[3, 0] = 0.0
    ref = torch.zeros(M, N)
    for kb in range(3):
        part = a[:, kb * 128:(kb + 1) * 128].float() @ b[:, kb * 128:(kb + 1) * 128].float().t()
        ref = ref + part * (sa[:, kb][:, None] * sb[:, kb][None, :])
    out = torch.empty(M, N, device=DEV, dtype=torch.float32)
    from mdy_triton_amd import _lib
    ad, bd, sad, sbd = a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV)
    rc = _lib.load().mdy_fp8_gemm_nt_rowscaled(ad.data_ptr(), sad.data_ptr(), 3, 1, bd.data_ptr(), sbd.data_ptr(), 3, 1,
                                                out.data_ptr(), M, N, K, 0, 1, None)
    torch.cuda.synchronize()
    assert rc == 0
    got = out.cpu()
    assert torch.equal(torch.isnan(got), torch.isnan(ref)) and torch.isnan(got[1]).all() and torch.isnan(got[:, 5]).all()
    assert torch.equal(torch.isinf(got), torch.isinf(ref)) and torch.equal(got[torch.isinf(ref)], ref[torch.isinf(ref)])
    fin = torch.isfinite(ref)
    assert fin[4:].any() and torch.allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-2)


def test_fp8_linear_reproduces_the_reference_notebook_error_magnitudes():
    """The one numeric record the reference keeps for this layer (deepseekv3/fp8-benchmark.ipynb cell 6, outputs at raw
    lines 195 / 216 / 236 / 256): Fp8Linear (e4m3fn) against a bf16 nn.Linear with the same parameters, bs = 4,
    seq = 4096, d = 4096, bias, x ~ randn, dy ~ rand: forward max / mean |error| 0.1172 / 0.0167, input gradient
    0.0669 / 0.0095, weight gradient 14.0 / 2.11, bias gradient allclose.  The data there is unseeded, so the
    statistics are what can be compared: a quantizer or GEMM that computed something else (another scale rule, a
    dropped K block, transposed scales) moves the means by far more than the 6 % bands below (measured here: 0.1172-0.125 / 0.0167, 0.0664-0.0669 / 0.0095,
    14.5-14.9 / 2.113)."""
    torch.manual_seed(0)
    bs, seq, d = 4, 4096, 4096
    x1 = torch.randn(bs, seq, d, dtype=torch.bfloat16, device=DEV).requires_grad_(True)
    x2 = x1.detach().clone().requires_grad_(True)
    fc1 = torch.nn.Linear(d, d, bias=True, device=DEV, dtype=torch.bfloat16)
    fc2 = m.Fp8Linear(d, d, bias=True, device=DEV, dtype=torch.bfloat16, fp8_dtype=torch.float8_e4m3fn)
    with torch.no_grad():
        fc2.weight.copy_(fc1.weight)
        fc2.bias.copy_(fc1.bias)
    y1, y2 = fc1(x1), fc2(x2)
    dy = torch.rand_like(y1)
    y1.backward(dy)
    y2.backward(dy)

    def err(a, b):
        e = (a.float() - b.float()).abs()
        return e.max().item(), e.mean().item()
    fmax, fmean = err(y1, y2)
    gmax, gmean = err(x1.grad, x2.grad)
    wmax, wmean = err(fc1.weight.grad, fc2.weight.grad)
    assert 0.94 * 0.0167 < fmean < 1.06 * 0.0167 and 0.5 * 0.1172 < fmax < 2 * 0.1172, (fmax, fmean)
    assert 0.94 * 0.0095 < gmean < 1.06 * 0.0095 and 0.5 * 0.0669 < gmax < 2 * 0.0669, (gmax, gmean)
    assert 0.94 * 2.11 < wmean < 1.06 * 2.11 and 0.5 * 14.0 < wmax < 2 * 14.0, (wmax, wmean)
    assert torch.allclose(fc1.bias.grad, fc2.bias.grad)


# ------------------------------------------------------------------ float8_e5m2: the reference's default fp8 dtype
E5M2 = torch.float8_e5m2


def test_e5m2_device_cast_matches_the_codec():
    """v_cvt_pk_bf8_f32 against the from-definition e5m2 codec on every code's neighbourhood and random values."""
    from oracle import fp8_format as F
    from mdy_triton_amd import _lib
    vals = F.decode_e5m2(np.arange(256, dtype=np.uint8))
    finite = np.sort(vals[np.isfinite(vals) & (vals >= 0)]).astype(np.float64)
    mids = (finite[:-1] + finite[1:]) / 2
    pts = []
    for v in np.concatenate([finite, mids]):
        f = np.float32(v)
        pts += [f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))]
    x = np.array(pts + [61439.0, 61440.0, 65536.0, 1e30], dtype=np.float32)
    rng = np.random.default_rng(1)
    x = np.concatenate([x, -x, (rng.standard_normal(200000) * 10.0 ** rng.integers(-6, 5, 200000)).astype(np.float32)])
    xt = torch.from_numpy(x).to(DEV)
    y = torch.empty(x.size, dtype=torch.uint8, device=DEV)
    _lib.check(_lib.load().mdy_cast_f32_to_e5m2(xt.data_ptr(), y.data_ptr(), x.size, None), "cast")
    assert np.array_equal(y.cpu().numpy(), F.encode_rne_e5m2(x))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_e5m2_quantizers_bit_exact(dtype):
    """act_quant_block (both directions) and weight_quant_block with the reference's DEFAULT dtype, float8_e5m2
    (fp8_kernel.py:62, 124): s = amax / 57344, bytes and scales bit-exact against the oracle."""
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(200, 384, generator=g) * 3).to(dtype)
    y, s = m.act_quant_block(x.to(DEV))                      # default dtype
    yr, sr = O.act_quant_block(x, dtype=E5M2)
    assert y.dtype == E5M2 and np.array_equal(u8(y), u8(yr)) and torch.equal(s.cpu(), sr)
    assert float(y.float().abs().max()) == 57344.0           # every group's largest element maps to the format's maximum
    yt, st = m.act_quant_block(x.to(DEV), transpose=True)
    ytr, str_ = O.act_quant_block(x, transpose=True, dtype=E5M2)
    assert yt.dtype == E5M2 and yt.shape == (384, 200) and np.array_equal(u8(yt), u8(ytr)) and torch.equal(st.cpu(), str_)
    w = (torch.randn(256, 384, generator=g) * 0.02).to(dtype)
    wq, ws = m.weight_quant_block(w.to(DEV))                 # default dtype
    wqr, wsr = O.weight_quant_block(w, dtype=E5M2)
    assert wq.dtype == E5M2 and np.array_equal(u8(wq), u8(wqr)) and torch.equal(ws.cpu(), wsr)
    wq4, _ = m.weight_quant_block(w.to(DEV), dtype=FP8)
    assert wq4.dtype == FP8


@pytest.mark.parametrize("M,N,K", [(128, 256, 256), (130, 200, 384), (256, 384, 1024), (2048, 3328, 256)])
def test_e5m2_gemms_exact_integer(M, N, K):
    """e5m2 operands through both GEMM forms of fp8_kernel.fp8_matmul (block-scaled weight: its scales expanded to one
    per row; row scales on both sides): integer operands and power-of-two scales are exact, so the result must equal
    the float64 computation rounded once to bf16."""
    g = torch.Generator().manual_seed(M + K)
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (N, K), generator=g)
    KB, NB = K // 128, (N + 127) // 128
    ea = torch.randint(-2, 3, (M, KB), generator=g)
    eb_blk = torch.randint(-2, 3, (NB, KB), generator=g)
    eb_row = torch.randint(-2, 3, (N, KB), generator=g)
    a, b = ai.float().to(E5M2).to(DEV), bi.float().to(E5M2).to(DEV)
    for have_w, eb in ((True, eb_blk), (False, eb_row)):
        if not have_w and M % 128:
            continue
        exact = torch.zeros(M, N, dtype=torch.float64)
        for kb in range(KB):
            sbn = eb[torch.arange(N) // 128, kb] if have_w else eb[:, kb]
            exact += (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()) * \
                torch.exp2((ea[:, kb][:, None] + sbn[None, :]).double())
        got = FK.fp8_matmul(a, b, torch.exp2(ea.float()).to(DEV), torch.exp2(eb.float()).to(DEV), have_w=have_w)
        assert torch.equal(got.cpu().double(), exact.to(torch.bfloat16).double()), have_w
    with pytest.raises(TypeError):
        FK.fp8_matmul(a, b.view(torch.uint8).view(FP8), torch.exp2(ea.float()).to(DEV), torch.exp2(eb_blk.float()).to(DEV))


@pytest.mark.parametrize("bias", [True, False])
def test_fp8_linear_e5m2_default(bias):
    """Fp8Linear as the reference constructs it by default (fp8_dtype = float8_e5m2): forward and all gradients within the
    GEMM tolerance of the oracle computing in e5m2."""
    g = torch.Generator().manual_seed(31)
    shape, N = (3, 100, 512), 384
    K = shape[-1]
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    b = torch.randn(N, generator=g).bfloat16() if bias else None
    x = torch.randn(*shape, generator=g).bfloat16()
    dy = torch.randn(*shape[:-1], N, generator=g).bfloat16()
    ref_out = O.fp8_linear_forward(x, w, b, dtype=E5M2)
    ref_dx, ref_dw, ref_db = O.fp8_linear_backward(x, w, dy, bias, dtype=E5M2)
    lin = m.Fp8Linear(K, N, bias=bias, dtype=torch.bfloat16)
    assert lin.fp8_dtype == E5M2
    with torch.no_grad():
        lin.weight.copy_(w)
        if bias:
            lin.bias.copy_(b)
    lin = lin.to(DEV)
    xg = x.to(DEV).requires_grad_(True)
    out = lin(xg)
    out.backward(dy.to(DEV))
    if bias:
        mag = torch.maximum(ref_out.float().abs(), (ref_out.float() - b.float()).abs())
        assert bool(((out.float().cpu() - ref_out.float()).abs() <= 2e-2 + 1e-2 * mag).all())
    else:
        assert close(out, ref_out)
    assert close(xg.grad, ref_dx) and close(lin.weight.grad, ref_dw)
    if bias:
        assert torch.allclose(lin.bias.grad.float().cpu(), ref_db.float(), rtol=1e-2, atol=1e-2)


def test_fp8_mlp_e5m2_default_paths_agree():
    """Fp8MLP with the reference's defaults (Fp8Linear projections, float8_e5m2): the three execution paths agree bit for
    bit, and the no-gradient result is within the GEMM tolerance of the oracle's composition stage by stage."""
    g = torch.Generator().manual_seed(41)
    H, inter = 256, 384
    x = torch.randn(64, H, generator=g).bfloat16()
    dy = torch.randn(64, H, generator=g).bfloat16()
    mlp = m.Fp8MLP(H, inter, device=DEV)
    assert mlp.fp8_dtype == E5M2 and mlp.up_gate_proj.fp8_dtype == E5M2
    outs = []
    for low in (False, True):
        mlp.zero_grad()
        xg = x.to(DEV).requires_grad_(True)
        y = mlp(xg, low_memory=low)
        y.backward(dy.to(DEV))
        outs.append((y.detach(), xg.grad, mlp.up_gate_proj.weight.grad.clone(), mlp.down_proj.weight.grad.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    with torch.no_grad():
        y0 = mlp(x.to(DEV))
        assert torch.equal(y0, outs[0][0])
        assert torch.equal(m.fp8_ckpt_mlp(x.to(DEV), mlp.up_gate_proj.weight, mlp.down_proj.weight), y0)   # reference defaults
        ug = mlp.up_gate_proj(x.to(DEV))
    assert close(ug, O.fp8_linear_forward(x, mlp.up_gate_proj.weight.detach().cpu(), None, dtype=E5M2))
    act = O.silu_fwd(ug.cpu(), "up-gate")
    assert close(y0, O.fp8_linear_forward(act, mlp.down_proj.weight.detach().cpu(), None, dtype=E5M2))


@pytest.mark.parametrize("M,N,K", [(256, 512, 256), (300, 520, 384), (2000, 2304, 1024), (4096, 1536, 1152), (1000, 1090, 1664),
                                   (520, 776, 1024), (512, 18432, 256)])
def test_e5m2_tile_kernels_exact_integer(M, N, K):
    """e5m2 operands on the tuned tile kernels (every tile configuration the dispatch picks for more than 64 rows): exact
    on integer operands with power-of-two scales, fp32 and bf16 output, with a bias in the epilogue."""
    from mdy_triton_amd import _lib
    g = torch.Generator().manual_seed(M + N + K)
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (N, K), generator=g)
    KB, NB = K // 128, (N + 127) // 128
    ae = torch.randint(-2, 3, (M, KB), generator=g)
    be = torch.randint(-2, 3, (NB, KB), generator=g)
    exact = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(KB):
        exact += (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()) * \
            torch.exp2((ae[:, kb][:, None] + be[torch.arange(N) // 128, kb][None, :]).double())
    a, b = ai.float().to(E5M2).to(DEV), bi.float().to(E5M2).to(DEV)
    a_s, b_s = torch.exp2(ae.float()).to(DEV), torch.exp2(be.float()).to(DEV)
    out = torch.full((M, N), float("nan"), device=DEV)
    L = _lib.load()
    assert L.mdy_fp8_gemm_nt_e5m2(a.data_ptr(), a_s.data_ptr(), KB, 1, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), None, M, N, K, 1,
                                  None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().double(), exact)
    bias = torch.randint(-8, 9, (N,), generator=g).float().bfloat16()
    got = FK.fp8_matmul(a, b, a_s, b_s, bias.to(DEV))
    assert torch.equal(got.cpu().double(), (exact + bias.double()).to(torch.bfloat16).double())
    # what the entry point does not take is refused, not mis-run: K not a multiple of 128, an unaligned operand
    assert L.mdy_fp8_gemm_nt_e5m2(a.data_ptr(), a_s.data_ptr(), KB, 1, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), None, M, N, K - 64, 1,
                                  None) == -2
    assert L.mdy_fp8_gemm_nt_e5m2(a.data_ptr() + 8, a_s.data_ptr(), KB, 1, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), None, M - 1, N, K,
                                  1, None) == -2


# (M, N, K) -> the branch of the <= 64-row dispatch it lands in
E5M2_SMALL = [(1, 512, 256), (5, 512, 384), (16, 520, 256), (17, 512, 256), (33, 512, 256), (64, 512, 256),      # whole-line kernel: 1, 2 and 4 row tiles, 16 columns per workgroup
              (48, 3600, 256), (64, 3200, 128), (48, 6400, 256), (64, 6404, 128),                                   # the same with 4 row tiles against a middling N
              (5, 16384, 256), (17, 9216, 256), (31, 9216, 128), (5, 25600, 256), (16, 25600, 128),                # 32 columns per workgroup
              (20, 25600, 256), (33, 25616, 256), (64, 25600, 128),                                                # strip kernel
              (48, 16384, 256), (33, 16400, 128),                                                                  # 128x128 tiles
              (48, 12800, 256), (64, 12804, 128)]                                                                  # 64x64 tiles


@pytest.mark.parametrize("M,N,K", E5M2_SMALL)
def test_e5m2_small_m_exact_integer(M, N, K):
    """e5m2 operands, up to 64 rows: every branch of the small-M dispatch (the whole-line kernel with 16 and 32 columns per
    workgroup and 1, 2 or 4 row tiles, the strip kernel, 128x128 and 64x64 tiles against a wide weight), exact on integer
    operands with power-of-two scales; fp32 and bf16 output, bias in the epilogue, through the C entry point and through
    fp8_matmul."""
    from mdy_triton_amd import _lib
    g = torch.Generator().manual_seed(7 * M + N + K)
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (N, K), generator=g)
    KB, NB = K // 128, (N + 127) // 128
    ae = torch.randint(-2, 3, (M, KB), generator=g)
    be = torch.randint(-2, 3, (NB, KB), generator=g)
    exact = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(KB):
        exact += (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()) * \
            torch.exp2((ae[:, kb][:, None] + be[torch.arange(N) // 128, kb][None, :]).double())
    a, b = ai.float().to(E5M2).to(DEV), bi.float().to(E5M2).to(DEV)
    a_s, b_s = torch.exp2(ae.float()).to(DEV), torch.exp2(be.float()).to(DEV)
    bias = torch.randint(-8, 9, (N,), generator=g).float().bfloat16()
    L = _lib.load()
    out = torch.full((M, N), float("nan"), device=DEV)
    assert L.mdy_fp8_gemm_nt_e5m2(a.data_ptr(), a_s.data_ptr(), KB, 1, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), None, M, N, K, 1,
                                  None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().double(), exact)
    # column-major activation scales (the layout quant_input returns), fp32 out with the bias
    a_st = a_s.t().contiguous()
    out = torch.full((M, N), float("nan"), device=DEV)
    bias_d = bias.to(DEV)
    assert L.mdy_fp8_gemm_nt_e5m2(a.data_ptr(), a_st.data_ptr(), 1, M, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), bias_d.data_ptr(), M,
                                  N, K, 1, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().double(), exact + bias.double())
    got = FK.fp8_matmul(a, b, a_s, b_s, bias_d)
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu().double(), (exact + bias.double()).to(torch.bfloat16).double())
    got = FK.fp8_matmul(a, b, a_s, b_s)
    assert torch.equal(got.cpu().double(), exact.to(torch.bfloat16).double())


def test_e5m2_small_m_realistic_against_oracle():
    """Decode-sized e5m2 GEMMs on quantized Gaussian data against the oracle's dequantize-then-matmul (rtol = atol = 1e-2)."""
    g = torch.Generator().manual_seed(99)
    for M, N, K in [(1, 7168, 2048), (16, 2048, 7168), (64, 7168, 2048), (40, 25600, 512)]:
        x = torch.randn(M, K, generator=g).bfloat16()
        w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
        xq, xs = O.act_quant_block(x, dtype=E5M2)
        wq, ws = O.weight_quant_block(w, dtype=E5M2)
        ref = O.fp8_gemm(xq, xs, wq, ws, dtype=torch.bfloat16)
        got = FK.fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV))
        assert close(got, ref), (M, N, K)


def test_act_quant_block_e5m2_golden_codes_on_device():
    """The closed-form e5m2 fixture on the device, both directions (the transposing kernel and the general row kernel)."""
    import os
    d = np.load(os.path.join(os.path.dirname(__file__), "golden", "act_quant_block_e5m2.npz"))
    x = torch.from_numpy(d["x_bits"].view(np.int16)).view(torch.bfloat16).to(DEV)
    y_t, s_t = m.act_quant_block(x, transpose=True)           # default dtype: float8_e5m2
    assert np.array_equal(u8(y_t), d["y_t"]) and np.array_equal(s_t.cpu().numpy(), d["s_t"])
    y, s = m.act_quant_block(x.t().contiguous())
    assert np.array_equal(u8(y), d["y_t"]) and np.array_equal(s.cpu().numpy(), d["s_t"])
