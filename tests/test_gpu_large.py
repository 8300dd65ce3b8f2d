"""Operands beyond 2^31 elements / 2^32 bytes: every kernel must address them with 64-bit offsets.
Inputs are generated on the device (they are too large to ship from the host); the oracle checks
slabs of rows at the start, across the 2^31-element / 2^32-byte boundary and at the end, and a
device-side restatement of the scale formula checks every scale."""
import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from oracle import oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
DEV = "cuda:0"
M_BIG, K_BIG = 36864, 65536          # 2.4e9 elements; element 2^31 is the first of row 32768


def u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def big_bf16(rows, cols, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV)
    for r in range(0, rows, 4096):
        x[r:r + 4096].normal_(generator=g)
        x[r:r + 4096] *= float(1 + (r // 4096) % 7)        # slabs differ in magnitude as well
    return x


H = 256                                # slab height (the training quantizers pad rows to 256)


def slabs(rows, boundary_row):
    """256-aligned slabs of H rows: first, the two around the boundary, last."""
    b = boundary_row // H * H
    return [0, b - H, b, rows - H]


@pytest.fixture(scope="module")
def x_big():
    x = big_bf16(M_BIG, K_BIG, 11)
    yield x
    del x
    torch.cuda.empty_cache()


def test_act_quant_beyond_2g_elements(x_big):
    y, s = m.act_quant(x_big)
    assert y.shape == x_big.shape and s.shape == (M_BIG, K_BIG // 128)
    # every scale: the group maximum comes from the device (exact), the IEEE division from the host
    for r in range(0, M_BIG, 8192):
        amax = x_big[r:r + 8192].view(-1, K_BIG // 128, 128).abs().amax(-1).float().cpu()
        assert torch.equal(s[r:r + 8192].cpu(), amax / 448.0), r
    for r in slabs(M_BIG, 32768):
        yr, sr = O.act_quant(x_big[r:r + H].cpu())
        assert np.array_equal(u8(y[r:r + H]), u8(yr)), r
        assert torch.equal(s[r:r + H].cpu(), sr), r


def test_training_quantizers_beyond_2g_elements(x_big):
    for fn, ofn in ((m.quant_input, lambda t: O.quant_input(t, only_forward=False)),
                    (m.quant_grad_output, O.quant_grad_output)):
        got = fn(x_big, only_forward=False) if fn is m.quant_input else fn(x_big)
        y, s, y_t, s_t = got
        assert y.shape == (M_BIG, K_BIG) and y_t.shape == (K_BIG, M_BIG)
        for r in slabs(M_BIG, 32768):
            yr, sr, ytr, str_ = ofn(x_big[r:r + H].cpu())
            assert np.array_equal(u8(y[r:r + H]), u8(yr)), r
            assert torch.equal(s[r:r + H].cpu(), sr), r
            assert np.array_equal(u8(y_t[:, r:r + H]), u8(ytr)), r
            # [K, M/128] (one scale per column and 128 rows) or [K/128, M/128] (one per 128x128 block)
            assert torch.equal(s_t[:, r // 128:(r + H) // 128].cpu(), str_), r
        del got, y, s, y_t, s_t
        torch.cuda.empty_cache()


def test_weight_quant_and_dequant_beyond_2g_elements(x_big):
    w = x_big                                              # any bf16 matrix with 128-aligned sides
    y, s = m.weight_quant_block(w, dtype=torch.float8_e4m3fn)
    assert s.shape == (M_BIG // 128, K_BIG // 128)
    for r in slabs(M_BIG, 32768):
        yr, sr = O.weight_quant_block(w[r:r + H].cpu())
        assert np.array_equal(u8(y[r:r + H]), u8(yr)), r
        assert torch.equal(s[r // 128:(r + H) // 128].cpu(), sr), r
    for dt in (torch.bfloat16, torch.float32):
        d = m.weight_dequant(y, s, out_dtype=dt)
        assert d.shape == w.shape and d.dtype == dt
        for r in slabs(M_BIG, 32768):
            dr = O.weight_dequant(y[r:r + H].cpu(), s[r // 128:(r + H) // 128].cpu(), dtype=dt)
            assert torch.equal(d[r:r + H].cpu(), dr), r
        # everything: the same fp32 product, rounded once to the output type, restated on the device
        for r in range(0, M_BIG, 4096):
            ref = (y[r:r + 4096].float().view(32, 128, K_BIG // 128, 128) *
                   s[r // 128:r // 128 + 32][:, None, :, None]).view(4096, K_BIG).to(dt)
            assert torch.equal(d[r:r + 4096], ref), r
        del d
        torch.cuda.empty_cache()


def test_fp8_gemm_operand_beyond_4g_bytes():
    """a is 66560 x 65536 bytes: byte 2^32 is the first of row 65536.  Small integers and power-of-two
    scales keep every sum exact in fp32, so slabs are compared bit for bit with an integer computation."""
    M, N, K = 66560, 256, 65536
    KB = K // 128
    g = torch.Generator(device=DEV).manual_seed(5)
    a = torch.empty(M, K, dtype=FP8, device=DEV)
    for r in range(0, M, 8192):
        a[r:r + 8192] = torch.randint(-2, 3, (min(8192, M - r), K), device=DEV, generator=g, dtype=torch.int8).float().to(FP8)
    b = torch.randint(-2, 3, (N, K), device=DEV, generator=g, dtype=torch.int8).float().to(FP8)
    ae = torch.randint(-1, 2, (M, KB), device=DEV, generator=g)
    be = torch.randint(-1, 2, (N // 128, KB), device=DEV, generator=g)
    c = m.fp8_gemm(a, torch.exp2(ae.float()), b, torch.exp2(be.float()), out_dtype=torch.float32)
    assert c.shape == (M, N)
    bd = b.cpu().float().double().view(N, KB, 128)
    for r in slabs(M, 65536):
        ad = a[r:r + H].cpu().float().double().view(H, KB, 128)
        part = torch.einsum("mkc,nkc->kmn", ad, bd)                          # [KB, H, N]
        e = ae[r:r + H].cpu().t()[:, :, None] + be.cpu()[torch.arange(N) // 128].t()[:, None, :]
        ref = (part * torch.exp2(e.double())).sum(0)
        assert torch.equal(c[r:r + H].cpu().double(), ref), r


def test_swiglu_beyond_4g_bytes(x_big):
    """The kernels are deterministic, so a slab of the large run must equal the same kernel run on that
    slab alone (the slab runs are what the small parity tests compare with the oracle)."""
    y, s, act = m.silu_act_quant(x_big, "gate-up", return_act=True)
    assert act.shape == (M_BIG, K_BIG // 2) and y.shape == act.shape and s.shape == (M_BIG, K_BIG // 256)
    assert torch.equal(act, m.silu_fwd(x_big, "gate-up"))
    dy = act                                               # any bf16 [M, N]
    dx = m.silu_bwd(dy, x_big, "gate-up")
    assert dx.shape == x_big.shape
    for r in slabs(M_BIG, 32768):
        xs = x_big[r:r + H].contiguous()
        ys, ss, acts = m.silu_act_quant(xs, "gate-up", return_act=True)
        assert torch.equal(act[r:r + H], acts), r
        assert np.array_equal(u8(y[r:r + H]), u8(ys)) and torch.equal(s[r:r + H], ss), r
        assert torch.equal(dx[r:r + H], m.silu_bwd(dy[r:r + H].contiguous(), xs, "gate-up")), r


# ---- more rows than grid.y could hold (65535 blocks): the kernels run on 1-D grids
def _row_samples(rows, h=64):
    return [0, rows // 2 // h * h, rows - h]


def test_act_quant_and_swiglu_with_a_million_rows():
    M, K = 64 * 65535 + 4104, 256                           # more rows than one launch of the row quantizers takes
    x = big_bf16(M, K, 31)
    y, s = m.act_quant(x)
    assert y.shape == (M, K) and s.shape == (M, 2)
    amax = x.view(M, 2, 128).abs().amax(-1).float().cpu()
    assert torch.equal(s.cpu(), amax / 448.0)
    for r in _row_samples(M):
        yr, sr = O.act_quant(x[r:r + 64].cpu())
        assert np.array_equal(u8(y[r:r + 64]), u8(yr)) and torch.equal(s[r:r + 64].cpu(), sr), r
    yq, sq, act = m.silu_act_quant(x, "up-gate", return_act=True)
    assert torch.equal(act, m.silu_fwd(x, "up-gate"))
    dx = m.silu_bwd(act, x, "up-gate")
    for r in _row_samples(M):
        xs = x[r:r + 64].contiguous()
        ys, ss, acts = m.silu_act_quant(xs, "up-gate", return_act=True)
        assert torch.equal(act[r:r + 64], acts), r
        assert np.array_equal(u8(yq[r:r + 64]), u8(ys)) and torch.equal(sq[r:r + 64], ss), r
        assert torch.equal(dx[r:r + 64], m.silu_bwd(acts, xs, "up-gate")), r


def test_weight_dequant_and_scalar_gemm_with_a_million_rows():
    N, K = 16 * 65535 + 272, 128                             # > 65535 blocks of 8 (dequant) and of 16 (GEMM) rows
    g = torch.Generator(device=DEV).manual_seed(41)
    q = torch.randint(-8, 9, (N, K), device=DEV, generator=g, dtype=torch.int8).float().to(FP8)
    s = torch.exp2(torch.randint(-2, 3, ((N + 127) // 128, 1), device=DEV, generator=g).float())
    d = m.weight_dequant(q, s, out_dtype=torch.float32)
    ref = q.float() * s.repeat_interleave(128, 0)[:N]
    assert torch.equal(d, ref)
    # K = 48 is not a multiple of 128: the one-thread-per-element kernel; small integers and power-of-two
    # scales make every sum exact
    Kg, Ng = 48, 24
    a = q[:, :Kg].contiguous()
    a_s = torch.exp2(torch.randint(-1, 2, (N, 1), device=DEV, generator=g).float())
    b = torch.randint(-4, 5, (Ng, Kg), device=DEV, generator=g, dtype=torch.int8).float().to(FP8)
    b_s = torch.full((1, 1), 0.5, device=DEV)
    c = m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.float32)
    ref = (a.float() @ b.float().t()) * a_s * 0.5
    assert torch.equal(c, ref)


def test_training_quantizers_with_more_than_65535_tile_rows():
    M, K = 128 * 65536, 256                                  # > 65535 tile rows of 128
    x = big_bf16(M, K, 51)
    y, s, y_t, s_t = m.quant_grad_output(x)
    assert y.shape == (M, K) and y_t.shape == (K, M)
    for r in slabs(M, M // 2):
        yr, sr, ytr, str_ = O.quant_grad_output(x[r:r + H].cpu())
        assert np.array_equal(u8(y[r:r + H]), u8(yr)) and torch.equal(s[r:r + H].cpu(), sr), r
        assert np.array_equal(u8(y_t[:, r:r + H]), u8(ytr)), r
        assert torch.equal(s_t[:, r // 128:(r + H) // 128].cpu(), str_), r
    del y, s, y_t, s_t
    wq, ws = m.weight_quant_block(x, dtype=torch.float8_e4m3fn)
    for r in slabs(M, M // 2):
        yr, sr = O.weight_quant_block(x[r:r + H].cpu())
        assert np.array_equal(u8(wq[r:r + H]), u8(yr)) and torch.equal(ws[r // 128:(r + H) // 128].cpu(), sr), r
