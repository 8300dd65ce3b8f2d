"""GPU parity of SwiGLU and of its fusion with the activation quantizer.

silu is floating point (exp / reciprocal differ between implementations by about one fp32 ulp), so the
bf16 activation is compared with the CPU oracle to within one bf16 ulp (rtol 2^-7) and the two must agree
bit for bit on all but a small fraction of elements; the quantizer part of the fused kernel is integer-exact:
its bytes and scales must equal the oracle quantizer applied to the kernel's own bf16 activation."""
import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from mdy_triton_amd import _lib
from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FP8 = torch.float8_e4m3fn
ULP = 2.0 ** -7      # one bf16 ulp, relative


def u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def up_gate(M, N2, seed, scale=2.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(M, N2, generator=g) * scale).bfloat16()


def within_ulp(got, ref, ulps=1):
    got, ref = got.float().cpu(), ref.float()
    ok = (got - ref).abs() <= ulps * ULP * ref.abs() + 1e-30
    same = (got == ref) | (got.isnan() & ref.isnan())
    return bool((ok | same).all()), float((~same).float().mean())


@pytest.mark.parametrize("order", ["up-gate", "gate-up"])
@pytest.mark.parametrize("M,N2", [(128, 512), (37, 1000), (4096, 4096), (5, 22)])
def test_silu_fwd(M, N2, order):
    x = up_gate(M, N2, M + N2)
    ok, frac = within_ulp(m.silu_fwd(x.to(DEV), order), O.silu_fwd(x, order))
    assert ok and frac < 2e-3


def test_silu_fwd_leading_dims_strides_and_extremes():
    x = up_gate(6 * 8, 512, 3).reshape(6, 8, 512)
    x[0, 0, :8] = torch.tensor([0.0, -0.0, 80.0, -80.0, 1e4, -1e4, 3e38, -3e38]).bfloat16()
    x[0, 0, 256:264] = torch.tensor([5.0, -5.0, 100.0, -100.0, -200.0, 200.0, 1.0, -1.0]).bfloat16()
    got = m.silu_fwd(x.to(DEV))
    assert got.shape == (6, 8, 256)
    ok, frac = within_ulp(got, O.silu_fwd(x))
    assert ok
    big = up_gate(40, 1024, 4)
    ok, _ = within_ulp(m.silu_fwd(big.to(DEV)[:, 256:768]), O.silu_fwd(big[:, 256:768]))     # row stride 1024
    assert ok
    assert m.silu_fwd(torch.empty(0, 256, dtype=torch.bfloat16, device=DEV)).shape == (0, 128)


@pytest.mark.parametrize("order", ["up-gate", "gate-up"])
@pytest.mark.parametrize("M,N2", [(128, 512), (33, 600), (2048, 4096)])
def test_silu_bwd_and_autograd(M, N2, order):
    x = up_gate(M, N2, M + 7)
    dy = up_gate(M, N2 // 2, M + 8, 1.0)
    ok, frac = within_ulp(m.silu_bwd(dy.to(DEV), x.to(DEV), order), O.silu_bwd(dy, x, order), ulps=2)
    assert ok and frac < 5e-3
    xg = x.to(DEV).requires_grad_(True)
    m.triton_silu(xg, order).backward(dy.to(DEV))
    ok, _ = within_ulp(xg.grad, O.silu_bwd(dy, x, order), ulps=2)
    assert ok


@pytest.mark.parametrize("order", ["up-gate", "gate-up"])
@pytest.mark.parametrize("M,N2", [(128, 512), (4096, 2 * 2048), (3, 256), (100, 2 * 18432)])
def test_silu_act_quant_official(M, N2, order):
    x = up_gate(M, N2, M + N2 + 1)
    y, s, act = m.silu_act_quant(x.to(DEV), order, return_act=True)
    ok, frac = within_ulp(act, O.silu_fwd(x, order))
    assert ok and frac < 2e-3
    y_ref, s_ref = O.act_quant(act.cpu())                       # the quantizer part is exact
    assert torch.equal(s.cpu(), s_ref) and np.array_equal(u8(y), u8(y_ref))
    y2, s2 = m.silu_act_quant(x.to(DEV), order)                 # same bytes when the activation is not written
    assert torch.equal(y2.view(torch.uint8), y.view(torch.uint8)) and torch.equal(s2, s)
    assert torch.equal(act, m.silu_fwd(x.to(DEV), order))
    # against the fully unfused oracle: scales within one bf16 ulp of the group maximum
    _, s_o, _ = O.silu_act_quant(x, order)
    assert torch.allclose(s.cpu(), s_o, rtol=ULP, atol=0)


def test_silu_act_quant_deeplinear_layout_and_zero_groups():
    x = up_gate(6, 2 * 300, 11)
    y, s, act = m.silu_act_quant(x.to(DEV), return_act=True, dialect="deeplinear")
    y_ref, s_ref, _, _ = O.quant_input(act.cpu(), True)
    assert y.shape == y_ref.shape == (8, 512) and s.shape == s_ref.shape and s.stride() == s_ref.stride()
    assert torch.equal(s.cpu(), s_ref) and np.array_equal(u8(y), u8(y_ref))
    # an all-zero group in the official dialect: s = 0, bytes NaN (as act_quant)
    z = torch.zeros(2, 512, dtype=torch.bfloat16)
    yz, sz = m.silu_act_quant(z.to(DEV))
    assert torch.count_nonzero(sz) == 0 and np.all((u8(yz) & 0x7F) == 0x7F)


def test_swiglu_abi_rejects_bad_arguments():
    L = _lib.load()
    x = torch.zeros(8, 512, dtype=torch.bfloat16, device=DEV)
    act = torch.empty(8, 256, dtype=torch.bfloat16, device=DEV)
    y = torch.empty(8, 256, dtype=torch.uint8, device=DEV)
    s = torch.empty(8, 2, dtype=torch.float32, device=DEV)
    assert L.mdy_swiglu(x.data_ptr(), None, None, None, 8, 256, 512, 0, 0, 0, 0, 0, 0, None) == -1
    assert L.mdy_swiglu(x.data_ptr(), None, y.data_ptr(), None, 8, 256, 512, 0, 8, 256, 2, 1, 0, None) == -1
    assert L.mdy_swiglu(x.data_ptr(), None, y.data_ptr(), s.data_ptr(), 8, 256, 512, 0, 8, 200, 2, 1, 0, None) == -2
    assert L.mdy_swiglu(x.data_ptr(), None, y.data_ptr(), s.data_ptr(), 8, 256, 512, 0, 8, 256, 2, 1, 7, None) == -4
    assert L.mdy_swiglu(x.data_ptr(), act.data_ptr(), None, None, 8, 256, 500, 0, 0, 0, 0, 0, 0, None) == -2
    assert L.mdy_swiglu_bwd(x.data_ptr(), None, x.data_ptr(), 8, 256, 512, 0, None) == -1
    with pytest.raises(AssertionError):
        m.silu_fwd(x, "gate_up")


# ------------------------------------------------------------------ Fp8MLP (fp8_kernel.py:436-515)
def _within(got, want):
    g_, w_ = got.float().cpu(), want.float()
    return bool(((g_ - w_).abs() <= 1e-2 + 1e-2 * w_.abs()).all())


@pytest.mark.parametrize("order", ["up-gate", "gate-up"])
@pytest.mark.parametrize("shape,inter", [((3, 100, 512), 768), ((256, 1024), 1280)])
def test_fp8_mlp_three_paths(shape, inter, order):
    """Composition with gradients, the memory-saving op and the gradient-free fused path agree bit for bit
    with each other (same kernels on the same values).  Against the CPU oracle every stage is held to the
    GEMM tolerance (rtol = atol = 1e-2) with the oracle fed the device's own bf16 intermediates; the chain
    as a whole cannot be held to it element by element (a one-ulp difference in up_gate or dact moves a few
    values across an e4m3fn rounding boundary, a 6 % step in that term of the next GEMM's sums), so end to
    end the bar is a relative Frobenius error below 0.5 %."""
    H = shape[-1]
    g = torch.Generator().manual_seed(inter + H)
    x = torch.randn(*shape, generator=g).bfloat16()
    w_ug = (torch.randn(2 * inter, H, generator=g) * 0.03).bfloat16()
    w_d = (torch.randn(H, inter, generator=g) * 0.03).bfloat16()
    dy = torch.randn(*shape, generator=g).bfloat16()

    mlp = m.Fp8MLP(H, inter, order=order, device=DEV, dialect="deeplinear", fp8_dtype=torch.float8_e4m3fn)
    up, down = mlp.up_gate_proj, mlp.down_proj
    with torch.no_grad():
        up.weight.copy_(w_ug)
        down.weight.copy_(w_d)
    results = []
    for low_memory in (False, True):
        mlp.zero_grad()
        xg = x.to(DEV).requires_grad_(True)
        y = mlp(xg, low_memory=low_memory)
        y.backward(dy.to(DEV))
        results.append((y.detach(), xg.grad, up.weight.grad.clone(), down.weight.grad.clone()))
    for a, b in zip(*results):
        assert a.shape == b.shape and a.dtype == torch.bfloat16 and torch.equal(a, b)
    with torch.no_grad():
        assert torch.equal(mlp(x.to(DEV)), results[0][0])
    mlp.low_memory = True                                        # the attribute switches the path as well
    assert torch.equal(mlp(x.to(DEV).requires_grad_(True)), results[0][0])
    y_d, dx_d, dwug_d, dwd_d = results[0]

    # the same composition by hand, keeping the intermediates
    mlp.zero_grad()
    xg = x.to(DEV).requires_grad_(True)
    ug_d = up(xg)
    ug_d.retain_grad()
    act_d = m.triton_silu(ug_d, order)
    act_d.retain_grad()
    y2 = down(act_d)
    y2.backward(dy.to(DEV))
    assert torch.equal(y2, y_d) and torch.equal(xg.grad, dx_d)
    ug_c, act_c = ug_d.detach().cpu(), act_d.detach().cpu()
    # stage by stage
    assert _within(ug_d, O.deep_linear_forward(x, w_ug, None))
    assert _within(y_d, O.deep_linear_forward(act_c, w_d, None))
    dact_r, dwd_r, _ = O.deep_linear_backward(act_c, w_d, dy, False)
    assert _within(act_d.grad, dact_r) and _within(dwd_d, dwd_r)
    dx_r, dwug_r, _ = O.deep_linear_backward(x, w_ug, ug_d.grad.cpu(), False)
    assert _within(dx_d, dx_r) and _within(dwug_d, dwug_r)
    # end to end
    up_gate = O.deep_linear_forward(x, w_ug, None)
    act = O.silu_fwd(up_gate, order)
    dact, dw_d_ref, _ = O.deep_linear_backward(act, w_d, dy, False)
    dx_ref, dw_ug_ref, _ = O.deep_linear_backward(x, w_ug, O.silu_bwd(dact, up_gate, order), False)
    for got, want in zip(results[0], (O.deep_linear_forward(act, w_d, None), dx_ref, dw_ug_ref, dw_d_ref)):
        assert got.shape == want.shape
        assert (got.float().cpu() - want.float()).norm() < 5e-3 * want.float().norm()


def test_fp8_ckpt_mlp_reference_call_order():
    """The reference calls `fp8_ckpt_mlp(h, w1, w2, self.fp8_dtype, self.order)` (fp8_kernel.py:510): the
    fourth positional argument is the fp8 dtype, the fifth the order; float8_e5m2 (the reference's default)
    is refused with a clear error."""
    g = torch.Generator().manual_seed(5)
    H, inter = 256, 384
    x = torch.randn(32, H, generator=g).bfloat16().to(DEV)
    w_ug = (torch.randn(2 * inter, H, generator=g) * 0.03).bfloat16().to(DEV)
    w_d = (torch.randn(H, inter, generator=g) * 0.03).bfloat16().to(DEV)
    mlp = m.Fp8MLP(H, inter, order="gate-up", device=DEV, dialect="deeplinear", fp8_dtype=torch.float8_e4m3fn)
    with torch.no_grad():
        mlp.up_gate_proj.weight.copy_(w_ug)
        mlp.down_proj.weight.copy_(w_d)
        want = mlp(x)
        got = m.fp8_ckpt_mlp(x, w_ug, w_d, torch.float8_e4m3fn, "gate-up", dialect="deeplinear")
        assert torch.equal(got, want)
        assert torch.equal(m.fp8_ckpt_mlp(x, w_ug, w_d, fp8_dtype=torch.float8_e4m3fn, order="gate-up", dialect="deeplinear"), want)
        with pytest.raises(TypeError, match="float8_e4m3fn"):
            m.fp8_ckpt_mlp(x, w_ug, w_d, torch.float8_e5m2, "gate-up", dialect="deeplinear")      # the DeepLinear dialect is e4m3fn only
        with pytest.raises(TypeError, match="float8_e4m3fn"):
            m.Fp8MLP(H, inter, fp8_dtype=torch.float8_e5m2, device=DEV, dialect="deeplinear")
        with pytest.raises(TypeError, match="float8_e4m3fn"):
            m.Fp8MLP(H, inter, fp8_dtype=torch.float16, device=DEV)


@pytest.mark.parametrize("order", ["up-gate", "gate-up"])
def test_fp8_mlp_official_dialect_three_paths(order):
    """The reference's own Fp8MLP (projections = Fp8Linear, s = amax / 448): composition with gradients, the
    memory-saving op (called positionally as the reference does) and the gradient-free fused path agree bit for bit;
    every stage is within the GEMM tolerance of the oracle fed the device's own bf16 intermediates."""
    H, inter, shape = 512, 768, (3, 100, 512)
    g = torch.Generator().manual_seed(77)
    x = torch.randn(*shape, generator=g).bfloat16()
    w_ug = (torch.randn(2 * inter, H, generator=g) * 0.03).bfloat16()
    w_d = (torch.randn(H, inter, generator=g) * 0.03).bfloat16()
    dy = torch.randn(*shape, generator=g).bfloat16()
    mlp = m.Fp8MLP(H, inter, order=order, device=DEV, fp8_dtype=torch.float8_e4m3fn)
    assert mlp.dialect == "official" and isinstance(mlp.up_gate_proj, m.Fp8Linear)
    up, down = mlp.up_gate_proj, mlp.down_proj
    with torch.no_grad():
        up.weight.copy_(w_ug)
        down.weight.copy_(w_d)
    results = []
    for low_memory in (False, True):
        mlp.zero_grad()
        xg = x.to(DEV).requires_grad_(True)
        y = mlp(xg, low_memory=low_memory)
        y.backward(dy.to(DEV))
        results.append((y.detach(), xg.grad, up.weight.grad.clone(), down.weight.grad.clone()))
    for a, b in zip(*results):
        assert a.shape == b.shape and a.dtype == torch.bfloat16 and torch.equal(a, b)
    with torch.no_grad():
        assert torch.equal(mlp(x.to(DEV)), results[0][0])
        assert torch.equal(m.fp8_ckpt_mlp(x.to(DEV), up.weight, down.weight, torch.float8_e4m3fn, order), results[0][0])
    y_d, dx_d, dwug_d, dwd_d = results[0]
    # stage by stage against the oracle
    mlp.zero_grad()
    xg = x.to(DEV).requires_grad_(True)
    ug_d = up(xg)
    ug_d.retain_grad()
    act_d = m.triton_silu(ug_d, order)
    act_d.retain_grad()
    y2 = down(act_d)
    y2.backward(dy.to(DEV))
    assert torch.equal(y2, y_d)
    ug_c, act_c = ug_d.detach().cpu(), act_d.detach().cpu()
    assert _within(ug_d, O.fp8_linear_forward(x, w_ug, None))
    assert _within(y_d, O.fp8_linear_forward(act_c, w_d, None))
    dact_r, dwd_r, _ = O.fp8_linear_backward(act_c, w_d, dy, False)
    assert _within(act_d.grad, dact_r) and _within(dwd_d, dwd_r)
    dx_r, dwug_r, _ = O.fp8_linear_backward(x, w_ug, ug_d.grad.cpu(), False)
    assert _within(dx_d, dx_r) and _within(dwug_d, dwug_r)


def test_megatron_swiglu_impl():
    """megatron_patchs/swiglu.py: swiglu_impl(x, bias, fp8_input_store) = silu(first half) * second half, with the
    matching gradient."""
    from mdy_triton_amd.megatron_patchs.swiglu import fused_up_gate_silu_no_split, swiglu_impl
    g = torch.Generator().manual_seed(4)
    x = torch.randn(3, 40, 512, generator=g).bfloat16()
    dy = torch.randn(3, 40, 256, generator=g).bfloat16()
    xg = x.to(DEV).requires_grad_(True)
    y = swiglu_impl(xg, None)
    y.backward(dy.to(DEV))
    ref = O.silu_fwd(x, "gate-up")
    assert y.shape == (3, 40, 256) and torch.allclose(y.float().cpu(), ref.float(), rtol=2 ** -7, atol=1e-6)
    dref = O.silu_bwd(dy, x, "gate-up")
    assert torch.allclose(xg.grad.float().cpu(), dref.float(), rtol=2 ** -6, atol=1e-3)
    assert torch.equal(fused_up_gate_silu_no_split(x.to(DEV), "gate-up"), y.detach())
