"""GPU parity of the grouped (mixture-of-experts) GEMM and the quantizers around it against the CPU oracle."""
import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from mdy_triton_amd import _lib
from oracle import oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu


def _single_pass_matmul(qa, sa, qb, sb):
    """The dense GEMM without a workspace (fp8_matmul may split this shape along K, which sums in another order)."""
    from mdy_triton_amd import _lib
    M, K = qa.shape
    N = qb.shape[0]
    out = torch.empty(M, N, device=qa.device, dtype=torch.bfloat16)
    _lib.check(_lib.load().mdy_fp8_gemm_nt(qa.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), qb.data_ptr(),
                                           sb.data_ptr(), out.data_ptr(), None, M, N, K, 0, None), "fp8_gemm_nt")
    torch.cuda.synchronize()
    return out
DEV = "cuda:0"
FP8 = torch.float8_e4m3fn
RTOL = ATOL = 1e-2     # the GEMM tolerance of the dense path


def u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def same(got, ref):
    assert got.shape == ref.shape and got.stride() == ref.stride()
    if ref.dtype == FP8:
        assert np.array_equal(u8(got), u8(ref))
    else:
        assert torch.equal(got.cpu().contiguous(), ref.contiguous())


def exact_grouped_case(m_splits, N, K, seed, device_call):
    """Integer operands and power-of-two scales: every product and partial sum is exact in fp32, so the
    result must equal the float64 computation bit for bit, group by group."""
    g = torch.Generator().manual_seed(seed)
    G, M = len(m_splits), sum(m_splits)
    KB, NB = K // 128, (N + 127) // 128
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (G, N, K), generator=g)
    ae = torch.randint(-2, 3, (M, KB), generator=g)
    be = torch.randint(-2, 3, (G, NB, KB), generator=g)
    ref = torch.zeros(M, N, dtype=torch.float64)
    row = 0
    for gi, mg in enumerate(m_splits):
        for kb in range(KB):
            part = ai[row:row + mg, kb * 128:(kb + 1) * 128].double() @ bi[gi, :, kb * 128:(kb + 1) * 128].double().t()
            ref[row:row + mg] += part * torch.exp2((ae[row:row + mg, kb][:, None] + be[gi, torch.arange(N) // 128, kb][None, :]).double())
        row += mg
    got = device_call(ai.float().to(FP8).to(DEV), torch.exp2(ae.float()).to(DEV), bi.float().to(FP8).to(DEV),
                      torch.exp2(be.float()).to(DEV), m_splits)
    assert torch.equal(got.cpu().double(), ref)


def call_f32(qa, sa, qb, sb, m_splits):
    """fp32 output through the C ABI (the Python wrapper returns bf16 like the reference)."""
    import ctypes
    M, K = qa.shape
    G, N, _ = qb.shape
    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.float32)
    arr = (ctypes.c_int64 * G)(*m_splits)
    _lib.check(_lib.load().mdy_fp8_grouped_gemm_nt(qa.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), qb.data_ptr(),
                                                   sb.data_ptr(), out.data_ptr(), None, ctypes.cast(arr, ctypes.c_void_p), G, N, K, 1,
                                                   None), "grouped")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("m_splits,N,K", [([256, 512, 0, 256], 520, 384),          # all multiples of 256: 256x256 tiles
                                          ([100, 0, 1, 300, 129, 128], 776, 256),  # ragged groups: 128x256 last tiles, tails everywhere
                                          ([384, 640, 129, 257, 0, 900, 128, 1], 776, 640),   # 256-row tiles + a 128-row last tile
                                          ([16] * 32, 2048, 512),                  # decode-like: many tiny groups
                                          ([3, 5], 40, 128)])
def test_grouped_gemm_exact_integer(m_splits, N, K):
    exact_grouped_case(m_splits, N, K, sum(m_splits) + N + K, call_f32)


@pytest.mark.parametrize("m_splits,N,K", [([1, 64, 0, 17, 33, 48, 16, 5], 3300, 896),    # ragged rows and columns, K tail step
                                          ([40] * 40, 640, 128),                          # one K block
                                          ([24] * 9, 3000, 2560),                         # 5 steps of 4 K blocks: odd number of steps
                                          ([64] * 4, 6400, 1152),                         # 49..64 rows: steps of 2 K blocks, 9 K blocks
                                          ([56] * 25, 1024, 128), ([50, 64] * 13, 1000, 256),     # the same with one K block / one step
                                          ([49] * 30, 900, 640)])
def test_grouped_gemm_exact_integer_strip_kernel(m_splits, N, K):
    """17..64 rows in the largest group and >= 200 strips of 128 columns: the weight-streaming strip kernel runs."""
    assert 16 < max(m_splits) <= 64 and len(m_splits) * ((N + 127) // 128) >= 200
    exact_grouped_case(m_splits, N, K, 3 * sum(m_splits) + N + K, call_f32)


@pytest.mark.parametrize("m_splits,N,K", [([1, 16, 0, 7, 3, 24, 9, 2], 3001, 896),        # one or two row tiles, ragged N, 7 K blocks
                                          ([16] * 40, 640, 128),                          # one K block: 7 of 8 waves idle
                                          ([2] * 64, 1030, 7168),                         # routed experts at decode, 7 K blocks per wave
                                          ([33, 64, 0, 40], 2050, 1152),                  # up to 64 rows, too few strips for the strip kernel
                                          ([30, 17, 32], 1000, 2176),                     # 17 K blocks: uneven shares of the waves
                                          ([5, 0, 0, 11], 290, 9344),                     # several passes over K
                                          ([12] * 3, 515, 3072), ([20, 4], 777, 5120)])   # pass depths that round up (3 -> 4, 5 -> 7 blocks)
def test_grouped_gemm_exact_integer_whole_line_kernel(m_splits, N, K):
    """At most 16 rows in the largest group, or at most 64 with fewer than 200 strips: every group is a small-M GEMM of
    the whole-line kernel (one grid row per group, empty groups return at once)."""
    strips = len(m_splits) * ((N + 127) // 128)
    assert max(m_splits) <= 16 or (max(m_splits) <= 64 and strips < 200)
    exact_grouped_case(m_splits, N, K, 5 * sum(m_splits) + N + K, call_f32)


def test_dense_wide_weight_exact_integer_strip_kernel():
    from tests.test_gpu_gemm import test_gemm_exact_integer_cases_all_kernels as dense_case
    dense_case(40, 25640, 640)       # 201 strips, 5 K blocks (two steps, the second partly past K), ragged N
    dense_case(5, 25600, 256)


def test_grouped_gemm_exact_integer_per_group_fallback():
    # more groups than the single-launch table holds, and K not a multiple of 128 is rejected by the MFMA path
    exact_grouped_case([2] * 300, 48, 128, 7, call_f32)


def test_grouped_matmul_against_oracle_with_bias_and_column_major_scales():
    G, N, K = 6, 1024, 2048
    m_splits = [256, 64, 0, 500, 1, 203]
    M = sum(m_splits)
    x = P.activations("outliers", M, K, 31)
    g = torch.Generator().manual_seed(32)
    ws = [(torch.randn(N, K, generator=g) * 0.02).bfloat16() for _ in range(G)]
    bias = torch.randn(G, N, generator=g).bfloat16()
    qa, sa, _, _ = m.per_token_cast_to_fp8(x.to(DEV))
    qb, sb = m.per_block_cast_to_fp8([w.to(DEV) for w in ws])
    assert qb.shape == (G, N, K) and sb.shape == (G, N // 128, K // 128) and sa.stride() == (1, qa.size(0))
    ra, rsa, _, _ = O.per_token_cast_to_fp8(x)
    rb, rsb = O.per_block_cast_to_fp8(ws)
    same(qa, ra); same(sa, rsa); same(qb, rb); same(sb, rsb)
    out = m.fp8_grouped_matmul(qa[:M], sa[:M], qb, sb, m_splits)
    ref = O.fp8_grouped_matmul(ra[:M], rsa[:M], rb, rsb, m_splits)
    assert out.dtype == torch.bfloat16 and out.shape == (M, N)
    assert torch.allclose(out.float().cpu(), ref.float(), rtol=RTOL, atol=ATOL)
    # decode-like split of the same rows (64 groups of 16: the whole-line small-M kernel, one grid row per group)
    small = [16] * 64
    Ms = sum(small)
    qb64, sb64 = qb.repeat(11, 1, 1)[:64].contiguous(), sb.repeat(11, 1, 1)[:64].contiguous()
    outs = m.fp8_grouped_matmul(qa[:Ms], sa[:Ms], qb64, sb64, small, bias=bias.repeat(11, 1)[:64].contiguous().to(DEV))
    refs = O.fp8_grouped_matmul(ra[:Ms], rsa[:Ms], rb.repeat(11, 1, 1)[:64], rsb.repeat(11, 1, 1)[:64], small,
                                bias=bias.repeat(11, 1)[:64])
    rows_s = torch.repeat_interleave(torch.arange(64), torch.tensor(small))
    mag_s = torch.maximum(refs.float().abs(), (refs.float() - bias.repeat(11, 1)[:64].float()[rows_s]).abs())
    assert bool(((outs.float().cpu() - refs.float()).abs() <= ATOL + RTOL * mag_s).all())
    outb = m.fp8_grouped_matmul(qa[:M], sa[:M], qb, sb, m_splits, bias=bias.to(DEV))
    refb = O.fp8_grouped_matmul(ra[:M], rsa[:M], rb, rsb, m_splits, bias=bias)
    rows = torch.repeat_interleave(torch.arange(G), torch.tensor(m_splits))
    mag = torch.maximum(refb.float().abs(), (refb.float() - bias.float()[rows]).abs())
    assert bool(((outb.float().cpu() - refb.float()).abs() <= ATOL + RTOL * mag).all())
    buf = torch.empty_like(out)
    assert m.fp8_grouped_matmul(qa[:M], sa[:M], qb, sb, m_splits, out=buf).data_ptr() == buf.data_ptr() and torch.equal(buf, out)
    # one group == the dense GEMM, bit for bit (same kernel body, same accumulation order)
    one = m.fp8_grouped_matmul(qa[:256], sa[:256], qb[:1], sb[:1], [256])
    assert torch.equal(one, _single_pass_matmul(qa[:256], sa[:256], qb[0], sb[0]))


@pytest.mark.parametrize("M,N,seed", [(256, 512, 0), (130, 300, 1), (1000, 256, 2)])
def test_per_token_cast_with_transpose_bit_exact(M, N, seed):
    x = P.activations("outliers", M, N, seed)
    for g_, r_ in zip(m.per_token_cast_to_fp8(x.to(DEV), True), O.per_token_cast_to_fp8(x, True)):
        same(g_, r_)


def test_group_per_token_cast_bit_exact():
    m_splits = [256, 0, 512, 256]
    x = P.activations("outliers", sum(m_splits), 768, 5)
    y, s, yts, sts = m.group_per_token_cast_to_fp8(x.to(DEV), m_splits)
    ry, rs, ryts, rsts = O.group_per_token_cast_to_fp8(x, m_splits)
    same(y, ry); same(s, rs)
    assert len(yts) == len(sts) == 4
    for a_, b_ in zip(yts + sts, ryts + rsts):
        same(a_, b_)
    with pytest.raises(AssertionError):
        m.group_per_token_cast_to_fp8(x.to(DEV), [100, 924])


@pytest.mark.parametrize("normal,transpose", [(True, False), (True, True), (False, True)])
def test_per_block_cast_bit_exact(normal, transpose):
    g = torch.Generator().manual_seed(9)
    ws = [(torch.randn(200, 300, generator=g) * 0.02).bfloat16() for _ in range(3)]
    got = m.per_block_cast_to_fp8([w.to(DEV) for w in ws], normal, transpose)
    ref = O.per_block_cast_to_fp8(ws, normal, transpose)
    assert len(got) == len(ref) == 2 * (int(normal) + int(transpose))
    for a_, b_ in zip(got, ref):
        same(a_, b_)
    single = m.per_block_cast_to_fp8(ws[0].to(DEV), normal, transpose)
    for a_, b_ in zip(single, O.per_block_cast_to_fp8(ws[0], normal, transpose)):
        same(a_, b_)


def test_grouped_abi_rejects_bad_arguments():
    import ctypes
    L = _lib.load()
    a = torch.zeros(256, 128, dtype=torch.uint8, device=DEV)
    s = torch.ones(256, 1, device=DEV)
    b = torch.zeros(2, 128, 128, dtype=torch.uint8, device=DEV)
    bs = torch.ones(2, 1, 1, device=DEV)
    c = torch.empty(256, 128, dtype=torch.bfloat16, device=DEV)
    ok = (ctypes.c_int64 * 2)(128, 128)
    neg = (ctypes.c_int64 * 2)(300, -44)
    args = lambda sp, **kw: [a.data_ptr(), s.data_ptr(), 1, 1, b.data_ptr(), bs.data_ptr(), kw.get("c", c.data_ptr()), None,
                             ctypes.cast(sp, ctypes.c_void_p) if sp is not None else None, 2, 128, 128, kw.get("dt", 0), None]
    assert L.mdy_fp8_grouped_gemm_nt(*args(ok)) == 0
    assert L.mdy_fp8_grouped_gemm_nt(*args(neg)) == -2
    assert L.mdy_fp8_grouped_gemm_nt(*args(None)) == -1
    assert L.mdy_fp8_grouped_gemm_nt(*args(ok, dt=5)) == -4
    assert L.mdy_fp8_grouped_gemm_nt(*args(ok, c=c.data_ptr() + 1)) == -3
    with pytest.raises(ValueError):
        m.fp8_grouped_matmul(a.view(FP8), s, b.view(FP8), bs, [100, 100])


def test_custom_manger_funnel_and_weight_cache():
    """CustomManger (megatron_patchs/manger.py): the classmethods are the package's operators, and
    get_fp8_weight re-quantizes a parameter only after set_first_micro_batch(p, True)."""
    from mdy_triton_amd.megatron_patchs.manger import CustomManger as CM
    g = torch.Generator().manual_seed(3)
    w = torch.nn.Parameter((torch.randn(256, 512, generator=g) * 0.02).bfloat16().to(DEV))
    CM.clear()
    first = CM.get_fp8_weight(w)
    ref = m.per_block_cast_to_fp8(w.detach(), output_transpose=True)
    assert len(first) == 4 and all(torch.equal(a.view(torch.uint8) if a.dtype == FP8 else a,
                                               b.view(torch.uint8) if b.dtype == FP8 else b) for a, b in zip(first, ref))
    with torch.no_grad():
        w.mul_(2)
    assert CM.get_fp8_weight(w)[0].data_ptr() == first[0].data_ptr()          # not marked: the cached copies
    CM.set_first_micro_batch(w, True)
    again = CM.get_fp8_weight(w)
    ref2 = m.per_block_cast_to_fp8(w.detach(), output_transpose=True)                  # re-quantized from the new weight ...
    assert torch.equal(again[1], ref2[1]) and torch.equal(again[0].view(torch.uint8), ref2[0].view(torch.uint8))
    assert CM.get_fp8_weight(w)[0].data_ptr() == again[0].data_ptr()          # ... and are cached again
    # a list of expert weights is keyed by its first member
    experts = [torch.nn.Parameter((torch.randn(256, 256, generator=g) * 0.02).bfloat16().to(DEV)) for _ in range(3)]
    qe = CM.get_fp8_weight(experts)
    assert qe[0].shape == (3, 256, 256) and experts[0] in CM.fp8_weight_map
    # the funnel
    x = torch.randn(64, 512, generator=g).bfloat16().to(DEV)
    qx, sx, _, _ = CM.per_token_cast_to_fp8(x)
    out = CM.fp8_matmul(qx[:64], sx[:64], again[0][:256], again[1][:2])
    assert torch.equal(out, m.fp8_matmul(qx[:64], sx[:64], again[0][:256], again[1][:2]))
    t = torch.arange(12, device=DEV).reshape(3, 4).t()                         # non-contiguous rows
    assert CM.fix_tensor_shape(t, 2).is_contiguous() and CM.fix_tensor_shape(t, 2).shape == (2, 3)
    CM.clear()
    assert not CM.fp8_weight_map


def test_grouped_gemm_exact_integer_random_splits():
    """Twelve seeded group tables (empty, tiny, ragged and 256-aligned experts mixed) against the exact integer
    reference: every expert starts a new tile row, its last tile row may be the 128-row kind, and no row of
    one expert may see another expert's weight."""
    rng = np.random.default_rng(77)
    for case in range(12):
        G = int(rng.integers(1, 9))
        m_splits = [int(rng.choice([0, 1, 17, 100, 128, 129, 200, 256, 257, 300, 384, 385, 512, 700])) for _ in range(G)]
        if sum(m_splits) == 0:
            m_splits[0] = 130
        N = int(rng.choice([128, 200, 256, 520, 776, 1024]))
        K = 128 * int(rng.integers(1, 6))
        exact_grouped_case(m_splits, N, K, 1000 + case, call_f32)


# ------------------------------------------------------------------ Fp8Padding / Fp8Unpadding (dpsk_grouped_linear.py:690-902)
@pytest.mark.parametrize("dtype,H", [(torch.bfloat16, 512), (torch.bfloat16, 7), (torch.uint8, 33), (torch.float32, 64)])
def test_group_padding_bit_exact_and_round_trip(dtype, H):
    """Every alignment path (16-, 2- and 1-byte pieces), empty groups, more groups than one launch takes."""
    from mdy_triton_amd.megatron_patchs.dpsk_grouped_linear import Fp8Padding, Fp8Unpadding, pad_groups, unpad_groups
    rng = np.random.default_rng(5)
    for m_splits in ([3, 0, 256, 257, 1, 511], [100], [0, 0], [int(v) for v in rng.integers(0, 40, 300)]):
        rows = sum(m_splits)
        if dtype == torch.uint8:
            x = torch.from_numpy(rng.integers(1, 255, (rows, H), dtype=np.uint8))
        else:
            x = torch.from_numpy(rng.standard_normal((rows, H)).astype(np.float32)).to(dtype)
        want, pads = O.fp8_padding(x, m_splits)
        with torch.no_grad():
            got, got_pads = Fp8Padding(len(m_splits))(x.to(DEV), m_splits)
        assert got_pads == pads and got.dtype == dtype and got.shape == want.shape
        assert torch.equal(got.cpu().contiguous().flatten().view(torch.uint8), want.contiguous().flatten().view(torch.uint8))
        with torch.no_grad():
            back = Fp8Unpadding(len(m_splits))(got, m_splits)
        assert torch.equal(back.cpu().contiguous().flatten().view(torch.uint8), x.contiguous().flatten().view(torch.uint8))
        assert torch.equal(back.cpu().contiguous().flatten().view(torch.uint8), O.fp8_unpadding(want, m_splits).contiguous().flatten().view(torch.uint8))
        # a destination full of garbage is overwritten everywhere (the padding rows are written, not assumed zero)
        assert torch.equal(pad_groups(x.to(DEV), m_splits, multiple=64).cpu().contiguous().flatten().view(torch.uint8),
                           O.fp8_padding(x, m_splits, 64)[0].contiguous().flatten().view(torch.uint8))
        assert torch.equal(unpad_groups(pad_groups(x.to(DEV), m_splits, 64), m_splits, 64).cpu().contiguous().flatten().view(torch.uint8), x.contiguous().flatten().view(torch.uint8))
    with pytest.raises(ValueError):
        pad_groups(torch.zeros(5, 4, device=DEV), [2, 2])
    with pytest.raises(AssertionError):
        Fp8Padding(3)(torch.zeros(4, 4, device=DEV), [2, 2])


def test_group_padding_autograd_pair_and_ragged_quantizer():
    """Each direction is the other's gradient, and a ragged batch reaches the grouped quantizer (which wants groups
    of multiples of 256 rows, fp8_matmul.py:227) through the padding: bytes and scales equal the oracle's on the
    oracle's padded copy."""
    from mdy_triton_amd.megatron_patchs.dpsk_grouped_linear import Fp8Padding, Fp8Unpadding
    g = torch.Generator().manual_seed(8)
    m_splits = [130, 0, 300, 17]
    H = 512
    x = torch.randn(sum(m_splits), H, generator=g).bfloat16()
    xg = x.to(DEV).requires_grad_(True)
    padded, pads = Fp8Padding(4)(xg, m_splits)
    w = torch.randn(sum(pads), H, generator=g).bfloat16().to(DEV)
    (padded.float() * w.float()).sum().backward()
    assert torch.equal(xg.grad.cpu(), O.fp8_unpadding(w.cpu(), m_splits))
    pg = padded.detach().clone().requires_grad_(True)
    out = Fp8Unpadding(4)(pg, m_splits)
    dy = torch.randn(sum(m_splits), H, generator=g).bfloat16().to(DEV)
    out.backward(dy)
    assert torch.equal(pg.grad.cpu(), O.fp8_padding(dy.cpu(), m_splits)[0])
    # ragged batch -> padded -> grouped quantizer with transposed copies
    y, s, yts, sts = m.group_per_token_cast_to_fp8(padded.detach(), pads)
    ry, rs, ryts, rsts = O.group_per_token_cast_to_fp8(O.fp8_padding(x, m_splits)[0], pads)
    assert torch.equal(y.cpu().contiguous().flatten().view(torch.uint8), ry.contiguous().flatten().view(torch.uint8)) and torch.equal(s.cpu(), rs)
    for a, b in zip(yts, ryts):
        assert torch.equal(a.cpu().contiguous().flatten().view(torch.uint8), b.contiguous().flatten().view(torch.uint8))
    for a, b in zip(sts, rsts):
        assert torch.equal(a.cpu().contiguous(), b.contiguous())
