"""GPU parity of the block-scaled FP8 GEMM and of DeepLinear against the CPU oracle.

Tolerance (from the benchmark definition): bf16 output within rtol 1e-2 / atol 1e-2 of
dequantize-then-fp32-matmul.  Exactly-representable cases must match bit for bit."""
import os

import numpy as np
import pytest
import torch

import mdy_triton_amd as m
from mdy_triton_amd import _lib
from oracle import oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
FP8 = torch.float8_e4m3fn
DEV = "cuda:0"
RTOL, ATOL = 1e-2, 1e-2


def close(got, ref):
    return torch.allclose(got.float().cpu(), ref.float(), rtol=RTOL, atol=ATOL)


def close_biased(got, ref, bias):
    """The GEMM tolerance applied where it belongs when a bias follows: the relative part is taken of the
    GEMM result before the bias (ref - bias), since a one-ulp difference there survives a cancelling bias."""
    if bias is None:
        return close(got, ref)
    ref = ref.float()
    mag = torch.maximum(ref.abs(), (ref - bias.float().cpu()).abs())
    return bool(((got.float().cpu() - ref).abs() <= ATOL + RTOL * mag).all())


def quantized_problem(kind, M, N, K, seed):
    x = P.activations(kind, M, K, seed)
    a, a_s = O.act_quant(x)
    _, wq, ws = P.weights(N, K, seed + 1000)
    return a, a_s, wq, ws


def test_gemm_golden_exact_bits():
    d = np.load(os.path.join(GOLD, "gemm_exact.npz"))
    a = torch.from_numpy(d["a"]).view(FP8).to(DEV)
    b = torch.from_numpy(d["b"]).view(FP8).to(DEV)
    a_s, b_s = torch.from_numpy(d["a_s"]).to(DEV), torch.from_numpy(d["b_s"]).to(DEV)
    c32 = m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.float32)
    assert np.array_equal(c32.cpu().numpy().view(np.uint32), d["c_f32"].view(np.uint32))
    c16 = m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16)
    assert np.array_equal(c16.cpu().view(torch.int16).numpy().view(np.uint16), d["c_bf16_bits"])


@pytest.mark.parametrize("M,N,K", [(256, 512, 256), (300, 520, 384), (65, 130, 128), (100, 257, 256), (70, 1100, 512),
                                   (512, 2304, 1024)])
def test_gemm_exact_integer_cases_all_kernels(M, N, K):
    """Integer-valued operands, power-of-two scales: every product and sum is exact, so the
    result must equal the int64 computation bit for bit (catches any indexing mistake:
    transposed scales, wrong n//128, K-block order, tile edges)."""
    g = torch.Generator().manual_seed(M + N + K)
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (N, K), generator=g)
    KB, NB = K // 128, (N + 127) // 128
    ae = torch.randint(-2, 3, (M, KB), generator=g)
    be = torch.randint(-2, 3, (NB, KB), generator=g)
    c = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(KB):
        part = (ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t())
        c += part * torch.exp2((ae[:, kb][:, None] + be[torch.arange(N) // 128, kb][None, :]).double())
    got = m.fp8_gemm(ai.float().to(FP8).to(DEV), torch.exp2(ae.float()).to(DEV), bi.float().to(FP8).to(DEV),
                     torch.exp2(be.float()).to(DEV), out_dtype=torch.float32)
    assert torch.equal(got.cpu().double(), c)


@pytest.mark.parametrize("M,N,K", [(896, 9300, 256), (880, 9344, 640),         # 128x128 tiles, 2 K blocks in LDS
                                   (2000, 2304, 256), (2048, 2200, 512),          # the same for a short K
                                   (2000, 2304, 1024), (4096, 1536, 1152), (1300, 5800, 2304),   # 128x256 tiles, ring of 3
                                   (4096, 1100, 1024), (4000, 1530, 1280), (3000, 1700, 1152), (3072, 1536, 2048),   # 128x192 tiles (wave columns straddle weight-scale blocks)
                                   (12800, 384, 1024),                                              # 128x256 tiles although they pad more
                                   (38400, 128, 1024), (36000, 100, 1280),       # 256x128 tiles, ring of 3
                                   (1536, 2048, 128), (1500, 2000, 1280),      # 128x128 tiles, ring of 4 K blocks
                                   (1024, 1100, 128), (1000, 1090, 1664),      # 128x64 tiles, ring of 6
                                   (200, 300, 128), (130, 70, 2304), (520, 776, 1024),    # 64x64 tiles, ring of 8
                                   (40, 16400, 256), (64, 6500, 384), (33, 7168, 1280)])  # 32..64 rows, wide weight
def test_gemm_exact_integer_few_tiles_configs(M, N, K):
    """Shapes with fewer than 200 tiles of 256x256 pick tile size and LDS ring depth by tile count; K runs
    from one K block (shorter than every ring) to more K blocks than the deepest ring, M and N ragged."""
    test_gemm_exact_integer_cases_all_kernels(M, N, K)


@pytest.mark.parametrize("M,N,K", [(4096, 1536, 7168), (4000, 1531, 1152), (2048, 3000, 1408), (3900, 1345, 1024)])
def test_gemm_exact_integer_producer_consumer_tiles(M, N, K):
    """The 128x192 producer / consumer kernel through the C entry point: column-major activation scales (the layout
    quant_input returns), a bias in the epilogue, bf16 and fp32 output, ragged M, N not a multiple of 4 (scalar stores),
    odd and even numbers of K blocks.  Exact on integer operands with power-of-two scales."""
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
    bias = torch.randint(-8, 9, (N,), generator=g).float().bfloat16()
    a, b = ai.float().to(FP8).to(DEV), bi.float().to(FP8).to(DEV)
    a_st, b_s, bias_d = torch.exp2(ae.float()).t().contiguous().to(DEV), torch.exp2(be.float()).to(DEV), bias.to(DEV)
    lib = _lib.load()
    assert lib.mdy_fp8_gemm_path(a.data_ptr(), b.data_ptr(), 1, M, M, N, K, 0) == 3
    for dtype, code in ((torch.float32, 1), (torch.bfloat16, 0)):
        out = torch.full((M, N), float("nan"), device=DEV, dtype=dtype)
        assert lib.mdy_fp8_gemm_nt(a.data_ptr(), a_st.data_ptr(), 1, M, b.data_ptr(), b_s.data_ptr(), out.data_ptr(), bias_d.data_ptr(),
                                   M, N, K, code, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().double(), (exact + bias.double()).to(dtype).double())


def _random_mid_shapes():
    g = torch.Generator().manual_seed(20250101)
    out = []
    for _ in range(28):
        M = int(torch.randint(65, 4200, (1,), generator=g))
        N = int(torch.randint(8, 3200, (1,), generator=g))
        K = 128 * int(torch.randint(1, 17, (1,), generator=g))
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("M,N,K", _random_mid_shapes())
def test_gemm_exact_integer_random_mid_shapes(M, N, K):
    """Randomly drawn (seeded) shapes in the range where the dispatch picks among the few-tile configurations (one-body and
    producer / consumer kernels, every ring depth, ragged M and N, 1 to 16 K blocks): exact on integer operands."""
    test_gemm_exact_integer_cases_all_kernels(M, N, K)


SPLIT_SHAPES = [(128, 1536, 4096), (100, 777, 4224), (256, 4096, 4096), (130, 1100, 5120),
                (130, 520, 6528), (300, 1536, 4480), (1000, 640, 8192),             # slabs of 9 / 12 and 11 / 11 K blocks, 3 and 8 tile rows
                (64, 2304, 4352), (48, 4096, 7168),                                 # 33..64 rows on 64x64 tiles
                # 33..64 rows against at most 2048 columns: the whole-line kernel over slabs of K (one or two K blocks per
                # wave and pass, several passes, ragged N with the scalar reduction, a slab count that does not divide K)
                (64, 2048, 4352), (40, 300, 8192), (33, 130, 4096), (50, 1536, 7168), (37, 2042, 8192), (64, 1024, 16384),
                (48, 256, 32768)]


@pytest.mark.parametrize("M,N,K", SPLIT_SHAPES)
def test_gemm_exact_integer_split_k(M, N, K):
    """Few rows against a long K: fp8_gemm hands the library a workspace and the shape runs split along K
    (64x64 tiles, 128x64 and 128x128 tiles on the producer / consumer kernel, or the whole-line kernel for up to 64 rows against a narrow weight; N % 4 != 0 takes
    the scalar reduction).  Exact operands stay exact."""
    assert _lib.load().mdy_fp8_gemm_workspace_bytes(M, N, K) >= 2 * M * N * 4
    test_gemm_exact_integer_cases_all_kernels(M, N, K)


def _raw_gemm(a, a_s, b, b_s, bias, dtype, ws, ws_bytes=None):
    M, K = a.shape
    N = b.shape[0]
    c = torch.full((M, N), float("nan"), device=DEV, dtype=dtype)
    code = 0 if dtype == torch.bfloat16 else 1
    lib = _lib.load()
    if ws == "plain":
        rc = lib.mdy_fp8_gemm_nt(a.data_ptr(), a_s.data_ptr(), K // 128, 1, b.data_ptr(), b_s.data_ptr(), c.data_ptr(),
                                 bias.data_ptr() if bias is not None else None, M, N, K, code, None)
    else:
        rc = lib.mdy_fp8_gemm_nt_ws(a.data_ptr(), a_s.data_ptr(), K // 128, 1, b.data_ptr(), b_s.data_ptr(), c.data_ptr(),
                                    bias.data_ptr() if bias is not None else None, M, N, K, code,
                                    ws.data_ptr() if ws is not None else None,
                                    (ws.numel() if ws is not None else 0) if ws_bytes is None else ws_bytes, None)
    torch.cuda.synchronize()
    return rc, c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(128, 1536, 7168), (100, 777, 4224), (64, 2048, 7168), (64, 2304, 7168), (45, 1000, 5120),
                                   (300, 1536, 4480)])
def test_gemm_split_k_against_oracle_and_plain_path(M, N, K, dtype):
    """Through the C ABI: with a workspace the result is within the GEMM tolerance of the oracle and of the
    single-pass kernel (another summation order), deterministic, and the bias is added once; without one, or
    with one that is too small, the call is the single-pass kernel bit for bit."""
    a, a_s, b, b_s = quantized_problem("outliers", M, N, K, seed=K + M)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(3)) * 0.5).bfloat16()
    ref = O.fp8_gemm(a, a_s, b, b_s, dtype=torch.float32) + bias.float()
    ad, asd, bd, bsd, biasd = a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), bias.to(DEV)
    need = _lib.load().mdy_fp8_gemm_workspace_bytes(M, N, K)
    assert need > 0
    ws = torch.empty(need, device=DEV, dtype=torch.uint8)
    rc, plain = _raw_gemm(ad, asd, bd, bsd, biasd, dtype, "plain")
    assert rc == 0
    ws.fill_(0xFF)                                         # stale contents must not matter
    rc, split = _raw_gemm(ad, asd, bd, bsd, biasd, dtype, ws)
    assert rc == 0
    assert close_biased(split, ref, bias) and close_biased(plain, ref, bias)
    assert torch.allclose(split.float(), plain.float(), rtol=RTOL, atol=ATOL)
    rc, again = _raw_gemm(ad, asd, bd, bsd, biasd, dtype, ws)
    assert rc == 0 and torch.equal(again, split)
    for small in (None, ws[:need - 16]):
        rc, fb = _raw_gemm(ad, asd, bd, bsd, biasd, dtype, small)
        assert rc == 0 and torch.equal(fb, plain)
    rc, _ = _raw_gemm(ad, asd, bd, bsd, biasd, dtype, ws[4:], need - 4)     # misaligned workspace
    assert rc == -3                                        # MDY_E_ALIGN


def test_gemm_exact_integer_random_shapes():
    """60 seeded random shapes through every dispatch path (streaming, strip, 64..256-wide tiles, rings, split K,
    scalar): exact operands, so any wrong index, stale LDS buffer or misplaced scale shows as a bit difference."""
    g = torch.Generator().manual_seed(2024)
    shapes = []
    for _ in range(60):
        M = int(torch.randint(1, 700, (1,), generator=g)) if torch.rand(1, generator=g) < 0.8 else int(torch.randint(700, 3000, (1,), generator=g))
        N = int(torch.randint(1, 3000, (1,), generator=g))
        K = 128 * int(torch.randint(1, 40, (1,), generator=g))
        if torch.rand(1, generator=g) < 0.1:
            K += int(torch.randint(1, 128, (1,), generator=g))          # ragged K: scalar kernel
        shapes.append((M, N, K))
    shapes += [(48, 26000, 256), (64, 16500, 512), (33, 6400, 4096), (5, 25700, 384),   # strip / wide-weight rules
               (20, 9300, 384), (31, 18433, 256), (8, 16390, 512), (16, 24576, 128)]    # two column groups per workgroup
    for M, N, K in shapes:
        gi = torch.Generator().manual_seed(M * 7 + N * 3 + K)
        ai = torch.randint(-2, 3, (M, K), generator=gi)
        bi = torch.randint(-2, 3, (N, K), generator=gi)
        KB, NB = (K + 127) // 128, (N + 127) // 128
        ae = torch.randint(-1, 2, (M, KB), generator=gi)
        be = torch.randint(-1, 2, (NB, KB), generator=gi)
        got = m.fp8_gemm(ai.float().to(FP8).to(DEV), torch.exp2(ae.float()).to(DEV), bi.float().to(FP8).to(DEV),
                         torch.exp2(be.float()).to(DEV), out_dtype=torch.float32).cpu().double()
        sa = torch.exp2(ae.double()).repeat_interleave(128, 1)[:, :K]
        sb = torch.exp2(be.double()).repeat_interleave(128, 0)[:N].repeat_interleave(128, 1)[:, :K]
        ref = (ai.double() * sa) @ (bi.double() * sb).t()
        assert torch.equal(got, ref), (M, N, K)


def test_ops_follow_torchs_current_stream():
    """The launches go to torch's current stream of the tensors' device: a chain issued under a side stream, after
    work that is still running on that stream, gives the same bits as on the default stream (the reference
    notebooks run under torch.cuda.set_stream)."""
    x = P.activations("normal", 256, 4096, 9).to(DEV)
    _, wq, ws = P.weights(1024, 4096, 10)
    wq, ws = wq.to(DEV), ws.to(DEV)
    xq0, xs0 = m.act_quant(x)
    c0 = m.fp8_gemm(xq0, xs0, wq, ws, out_dtype=torch.bfloat16)        # this shape is split along K: workspace too
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    big = torch.randn(8192, 8192, device=DEV)
    with torch.cuda.stream(side):
        x2 = x.clone()
        for _ in range(4):
            big = big @ big * 1e-4                                       # keeps the side stream busy
        x2 = x2 + 0                                                     # produced on the side stream, behind the matmuls
        xq1, xs1 = m.act_quant(x2)
        c1 = m.fp8_gemm(xq1, xs1, wq, ws, out_dtype=torch.bfloat16)
    side.synchronize()
    assert torch.equal(xq1.view(torch.uint8), xq0.view(torch.uint8)) and torch.equal(xs1, xs0) and torch.equal(c1, c0)


def test_gemm_transposed_scale_scratch_is_bit_identical():
    """Big shapes with row-major activation scales and a workspace run the same tile kernels on a transposed copy of
    the scales: only addresses change, so the result equals the single-call path bit for bit (ragged M, bias)."""
    M, N, K = 4000, 7200, 7168
    g = torch.Generator().manual_seed(77)
    a = torch.randint(0, 120, (M, K), generator=g, dtype=torch.uint8).view(FP8).to(DEV)
    b = torch.randint(0, 120, (N, K), generator=g, dtype=torch.uint8).view(FP8).to(DEV)
    a_s = (torch.rand(M, K // 128, generator=g) * 1e-3 + 1e-3).to(DEV)
    b_s = (torch.rand((N + 127) // 128, K // 128, generator=g) * 1e-3 + 1e-3).to(DEV)
    bias = torch.randn(N, generator=g).bfloat16().to(DEV)
    need = _lib.load().mdy_fp8_gemm_workspace_bytes(M, N, K)
    assert 0 < need < 2 * M * (K // 128) * 4
    ws = torch.full((need,), 0xFF, device=DEV, dtype=torch.uint8)
    for dtype in (torch.bfloat16, torch.float32):
        rc0, plain = _raw_gemm(a, a_s, b, b_s, bias, dtype, "plain")
        rc1, with_ws = _raw_gemm(a, a_s, b, b_s, bias, dtype, ws)
        assert rc0 == 0 and rc1 == 0 and torch.equal(plain, with_ws)
        assert not torch.isnan(with_ws.float()).any()


def test_gemm_workspace_query():
    lib = _lib.load()
    big = lib.mdy_fp8_gemm_workspace_bytes(4096, 18432, 7168)            # fills the GPU: never split, but room for
    assert 4096 * 56 * 4 <= big < 4096 * 56 * 4 + 256                    # the transposed activation scales
    assert lib.mdy_fp8_gemm_workspace_bytes(4096, 1536, 7168) == 0       # too short a GEMM for that to pay
    assert lib.mdy_fp8_gemm_workspace_bytes(32, 7168, 16384) == 0        # weight-streaming kernel
    assert lib.mdy_fp8_gemm_workspace_bytes(128, 7168, 2048) == 0        # K too short to cut
    assert lib.mdy_fp8_gemm_workspace_bytes(128, 7168, 5000) == 0        # ragged K: scalar kernel
    assert lib.mdy_fp8_gemm_workspace_bytes(0, 7168, 16384) == 0 and lib.mdy_fp8_gemm_workspace_bytes(-1, 1, 1) == 0
    n = lib.mdy_fp8_gemm_workspace_bytes(128, 7168, 16384)
    assert n > 0 and n % (128 * 7168 * 4) == 0


@pytest.mark.parametrize("M,N,K", [(4000, 4328, 256), (3590, 4608, 384), (4096, 4352, 128), (4000, 2400, 256)])
def test_gemm_exact_integer_big_tiles_and_split_launch(M, N, K):
    """>= 200 tiles of 256x256: the big-tile kernel runs, and because the tile count is not a multiple
    of the CU count the last tile columns go to a second launch with 128x256 tiles (ragged M and N edges
    in both).  The last shape has 160 tiles of 256x256 (more 128x128 tiles than fit in one round): one
    partly filled round of the big tile."""
    test_gemm_exact_integer_cases_all_kernels(M, N, K)


def test_gemm_split_launch_with_bias_bf16():
    M, N, K = 4096, 4352, 256
    a, a_s, wq, ws = quantized_problem("normal", M, N, K, 21)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(3)).bfloat16()
    rows = torch.arange(0, M, 61)
    ref = O.fp8_gemm(a[rows].contiguous(), a_s[rows].contiguous(), wq, ws, dtype=torch.bfloat16, bias=bias)
    got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16, bias=bias.to(DEV))
    assert close_biased(got[rows.to(DEV)], ref, bias)


def test_gemm_is_deterministic_and_k_tail_blocks_are_not_touched():
    """Copies and prefetch touches that run past the last K block must go nowhere: the same call repeated
    gives identical bits, and a weight with a single K block works on every tile shape."""
    a, a_s, wq, ws = quantized_problem("normal", 4096, 4352, 128, 5)
    args = (a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV))
    first = m.fp8_gemm(*args, out_dtype=torch.float32)
    for _ in range(3):
        assert torch.equal(m.fp8_gemm(*args, out_dtype=torch.float32), first)
    ref = O.fp8_gemm(a[::97].contiguous(), a_s[::97].contiguous(), wq, ws, dtype=torch.float32)
    assert torch.allclose(first[::97].cpu(), ref, rtol=2e-3, atol=1e-3)
    test_gemm_exact_integer_cases_all_kernels(300, 520, 128)      # 128x128 tiles, one K block


@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
def test_gemm_small_m_exact(M):
    test_gemm_exact_integer_cases_all_kernels(M, 272, 384)


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
@pytest.mark.parametrize("M,N,K", [(1, 2048, 7168), (1, 7168, 2048), (2, 1000, 4096), (3, 259, 128), (4, 7001, 1024), (4, 520, 16384),
                                   (1, 33, 1664), (2, 4096, 3072), (1, 777, 8192), (1, 1000, 16384), (1, 2050, 4224)])
def test_gemm_row_vector_kernel_exact_integer(M, N, K, fmt):
    """One row against a K of 4224..16384 runs on the row-vector kernel (no matrix cores, one weight row per wave); the
    other shapes here (2..4 rows, short K) run on the whole-line MFMA kernel with a mostly empty row tile: exact on
    integer operands with power-of-two scales through the C entry points, row- and column-major activation scales, bias,
    fp32 and bf16 output, N not a multiple of the rows per workgroup, both fp8 formats; K beyond the row-vector kernel's
    LDS staging (16384) goes to an MFMA kernel and gives the same exact result."""
    _small_m_exact_through_c_abi(M, N, K, fmt, longer_k=(fmt == "e4m3fn"))


def test_gemm_whole_line_kernel_long_k_exact_integer():
    """Up to 64 rows against K > 65536 (beyond the tile kernels' 32-bit addressing): the whole-line kernel takes it in
    many passes; exact on integer operands."""
    test_gemm_exact_integer_cases_all_kernels(8, 48, 65536 + 512)
    test_gemm_exact_integer_cases_all_kernels(40, 80, 65536 + 128)


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
@pytest.mark.parametrize("M,N,K", [(16, 2048, 7168), (16, 7168, 2048), (5, 272, 128), (8, 1000, 1024), (9, 6401, 3072),
                                   (12, 1536, 1536), (16, 530, 4096), (13, 6500, 5120), (7, 333, 6144), (16, 4096, 8192),
                                   (11, 520, 16384), (16, 300, 18432), (6, 290, 9344), (15, 7000, 2176),
                                   (17, 2048, 7168), (32, 7168, 2048), (24, 777, 1024), (31, 6410, 2176), (20, 515, 3072),
                                   (32, 1000, 4096), (25, 300, 16384), (32, 290, 9344),
                                   (64, 7168, 2048), (33, 3201, 1024), (48, 6402, 4096), (64, 3300, 2176), (50, 4099, 128),
                                   (16, 32768, 512), (9, 16500, 512), (16, 24576, 1536), (3, 22000, 384),                    # short K against a large
                                   (16, 33000, 256), (2, 32768, 256), (13, 65540, 128), (1, 70000, 128),                      # weight: 2, 4 or 8 column sets
                                   (16, 6500, 4096), (4, 6404, 4224)])                                                        # passes of 4 / 5 blocks, registers held to 128
def test_gemm_whole_line_kernel_exact_integer(M, N, K, fmt):
    """5..32 rows, and up to 64 against a middling N, run on the whole-line kernel (one, two or four 16-row activation
    tiles, 16 or 32 weight columns per workgroup by N, 1..8 K blocks per wave and pass by K, several passes for long K,
    K-block counts that are no multiple of the 8 waves so that some waves get fewer blocks or none): exact on integer
    operands with power-of-two scales through the C entry points, row- and column-major activation scales, bias, fp32
    and bf16 output, ragged N, both fp8 formats."""
    _small_m_exact_through_c_abi(M, N, K, fmt, longer_k=False)


def _small_m_exact_through_c_abi(M, N, K, fmt, longer_k):
    dt = FP8 if fmt == "e4m3fn" else torch.float8_e5m2
    lib = _lib.load()
    entry = lib.mdy_fp8_gemm_nt if fmt == "e4m3fn" else lib.mdy_fp8_gemm_nt_e5m2
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
    bias = torch.randint(-8, 9, (N,), generator=g).float().bfloat16()
    a, b = ai.float().to(dt).to(DEV), bi.float().to(dt).to(DEV)
    a_s, b_s, bias_d = torch.exp2(ae.float()).to(DEV), torch.exp2(be.float()).to(DEV), bias.to(DEV)
    a_st = a_s.t().contiguous()
    for dtype, code in ((torch.float32, 1), (torch.bfloat16, 0)):
        for scales, rs, cs in ((a_s, KB, 1), (a_st, 1, M)):
            for bp, want in ((None, exact), (bias_d, exact + bias.double())):
                out = torch.full((M, N), float("nan"), device=DEV, dtype=dtype)
                assert entry(a.data_ptr(), scales.data_ptr(), rs, cs, b.data_ptr(), b_s.data_ptr(), out.data_ptr(),
                             bp.data_ptr() if bp is not None else None, M, N, K, code, None) == 0
                torch.cuda.synchronize()
                assert torch.equal(out.cpu().double(), want.to(dtype).double())
    if longer_k:              # a longer K than the kernel stages: the MFMA kernel, same exact result
        K2 = 16384 + 128
        a2 = torch.zeros(M, K2, dtype=torch.uint8, device=DEV).view(dt)
        b2 = torch.zeros(N, K2, dtype=torch.uint8, device=DEV).view(dt)
        a2[:, :K] = a
        b2[:, :K] = b
        a2_s = torch.ones(M, K2 // 128, device=DEV)
        b2_s = torch.ones(NB, K2 // 128, device=DEV)
        a2_s[:, :KB] = a_s
        b2_s[:, :KB] = b_s
        out = torch.full((M, N), float("nan"), device=DEV)
        assert entry(a2.data_ptr(), a2_s.data_ptr(), K2 // 128, 1, b2.data_ptr(), b2_s.data_ptr(), out.data_ptr(), None, M, N, K2, 1,
                     None) == 0
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().double(), exact)


def test_gemm_row_vector_kernel_against_oracle():
    """The row-vector kernel on quantized Gaussian data: within rtol = atol = 1e-2 of the oracle (it adds a K block in
    eight scaled parts, another rounding than the MFMA kernels), and within 2^-8 of the float64 truth's scale."""
    for M, N, K in [(1, 2048, 7168), (1, 7168, 2048), (4, 1536, 4096)]:
        a, a_s, wq, ws = quantized_problem("normal", M, N, K, seed=M + K)
        ref = O.fp8_gemm(a, a_s, wq, ws, dtype=torch.float32)
        got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV), out_dtype=torch.float32)
        assert close(got, ref)
        truth = O.fp8_gemm_f64(a, a_s, wq, ws)
        assert (got.cpu().double() - truth).abs().max() <= 2 ** -12 * truth.abs().max() + 1e-6


def test_gemm_one_hot_and_scale_block_perturbation():
    N, K = 512, 512
    g = torch.Generator().manual_seed(2)
    b = torch.randint(0, 0x77, (N, K), generator=g, dtype=torch.uint8).view(FP8)
    b_s = torch.rand(4, 4, generator=g) + 0.5
    M = 128
    a = torch.zeros(M, K).to(FP8)
    hot = torch.randint(0, K, (M,), generator=g)
    a.view(torch.uint8)[torch.arange(M), hot] = 0x38  # 1.0
    a_s = torch.rand(M, 4, generator=g) + 0.5
    c = m.fp8_gemm(a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32).cpu()
    bd = O.weight_dequant(b, b_s, dtype=torch.float32)
    expect = bd[:, hot].t() * a_s[torch.arange(M), hot // 128][:, None]
    assert torch.allclose(c, expect, rtol=1e-6, atol=0)
    b_s2 = b_s.clone(); b_s2[2, 1] *= 4
    a2 = torch.randint(0, 0x60, (M, K), generator=g, dtype=torch.uint8).view(FP8)
    a2_s = torch.ones(M, 4)
    d = (m.fp8_gemm(a2.to(DEV), a2_s.to(DEV), b.to(DEV), b_s2.to(DEV), out_dtype=torch.float32)
         - m.fp8_gemm(a2.to(DEV), a2_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32)).cpu()
    assert torch.count_nonzero(d[:, :256]) == 0 and torch.count_nonzero(d[:, 384:]) == 0
    assert torch.count_nonzero(d[:, 256:384]) > 0


def test_gemm_c1_cpu_reference_config_full():
    kind, M, N, K = P.CONFIGS["C1_cpu_reference"]
    a, a_s, wq, ws = quantized_problem(kind, M, N, K, 0)
    ref = O.fp8_gemm(a, a_s, wq, ws, dtype=torch.bfloat16)
    got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    assert close(got, ref)
    truth = O.fp8_gemm_f64(a, a_s, wq, ws)
    assert (got.cpu().double() - truth).abs().max() <= 2 ** -8 * truth.abs().max() + 1e-6


@pytest.mark.parametrize("name", ["C2_q_a_proj", "C3_mlp_up_gate", "C4_mlp_down"])
def test_gemm_full_size_configs_whole_matrix(name):
    """Full-size GEMM on the device against the oracle's dequantize + fp32 matmul of the WHOLE problem (about a
    second of CPU time per configuration), every element within rtol = atol = 1e-2.  The activations are
    quantized by the HIP act_quant (itself bit-exact against the oracle, asserted here too), so the GEMM is fed
    what the path really produces."""
    kind, M, N, K = P.CONFIGS[name]
    x = P.activations(kind, M, K, 10)
    _, wq, ws = P.weights(N, K, 1010)
    a_ref, as_ref = O.act_quant(x)
    a, a_s = m.act_quant(x.to(DEV))
    assert torch.equal(a.cpu().view(torch.uint8), a_ref.view(torch.uint8)) and torch.equal(a_s.cpu(), as_ref)
    got = m.fp8_gemm(a, a_s, wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16)
    ref = O.fp8_gemm(a_ref, as_ref, wq, ws, dtype=torch.bfloat16)
    assert got.shape == ref.shape == (M, N)
    err = (got.float().cpu() - ref.float()).abs()
    assert bool((err <= ATOL + RTOL * ref.float().abs()).all()), "max abs error %g" % float(err.max())
    del ref, err
    # linearity in the activation scales (size-independent property): doubling a_s doubles C exactly
    got2 = m.fp8_gemm(a, a_s * 2, wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16)
    assert torch.equal(got2, got * 2)


@pytest.mark.parametrize("M,N,K", P.DECODE_SHAPES)
def test_gemm_decode_shapes(M, N, K):
    """All six decode / routed-expert shapes, end to end on the device: the HIP act_quant quantizes the
    activation rows (bit-exact against the oracle) and its output feeds the GEMM."""
    x = P.activations("normal", M, K, M)
    _, wq, ws = P.weights(N, K, M + 1000)
    a_ref, as_ref = O.act_quant(x)
    a, a_s = m.act_quant(x.to(DEV))
    assert torch.equal(a.cpu().view(torch.uint8), a_ref.view(torch.uint8)) and torch.equal(a_s.cpu(), as_ref)
    ref = O.fp8_gemm(a_ref, as_ref, wq, ws, dtype=torch.bfloat16)
    got = m.fp8_gemm(a, a_s, wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16)
    assert close(got, ref)
    truth = O.fp8_gemm_f64(a_ref, as_ref, wq, ws)
    assert (got.cpu().double() - truth).abs().max() <= 2 ** -8 * truth.abs().max() + 1e-6


@pytest.mark.parametrize("M,N,K", [(5, 1536, 1536), (24, 2112, 7168), (32, 4096, 4096), (48, 3328, 2048),      # whole-line kernel: 1, 2, 4 row tiles
                                   (8, 25728, 512),                                                             # 32 columns per workgroup, wide N
                                   (40, 25600, 1024), (20, 25728, 640),                                         # strip kernel
                                   (9, 300, 9344)])                                                             # several passes over K
def test_gemm_small_m_kernels_against_oracle(M, N, K):
    """The small-M kernels on quantized Gaussian activations and weights (not only exact-integer operands): within the
    GEMM tolerance of the oracle's dequantize + fp32 matmul, and within 2^-8 of the float64 result's scale."""
    a, a_s, wq, ws = quantized_problem("normal", M, N, K, seed=M + N + K)
    ref = O.fp8_gemm(a, a_s, wq, ws, dtype=torch.bfloat16)
    got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16)
    assert close(got, ref)
    truth = O.fp8_gemm_f64(a, a_s, wq, ws)
    assert (got.cpu().double() - truth).abs().max() <= 2 ** -8 * truth.abs().max() + 1e-6


def test_gemm_scalar_fallback_warns_for_large_aligned_shapes():
    """K > 65536 with more than 64 rows runs on the one-thread-per-output kernel: correct, but the wrapper says so
    (once per shape); K % 128 != 0, the kernel's intended use, stays silent."""
    import warnings
    M, N, K = 80, 48, 65536 + 128
    g = torch.Generator().manual_seed(9)
    a = torch.randint(0, 0x60, (M, K), generator=g, dtype=torch.uint8).view(FP8)
    b = torch.randint(0, 0x60, (N, K), generator=g, dtype=torch.uint8).view(FP8)
    a_s = torch.rand(M, K // 128, generator=g) * 1e-2
    b_s = torch.rand(1, K // 128, generator=g) * 1e-2
    lib = _lib.load()
    assert lib.mdy_fp8_gemm_path(None, None, K // 128, 1, M, N, K, 1) == 0
    assert lib.mdy_fp8_gemm_path(None, None, 56, 1, 4096, 18432, 7168, 1) == 3
    with pytest.warns(RuntimeWarning, match="scalar fallback"):
        got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32)
    ref = O.fp8_gemm(a, a_s, b, b_s, dtype=torch.float32)
    assert torch.allclose(got.cpu(), ref, rtol=1e-3, atol=1e-5)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        m.fp8_gemm(a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32)      # warned once already
        m.fp8_gemm(a[:, :200].contiguous().to(DEV), a_s[:, :2].contiguous().to(DEV), b[:, :200].contiguous().to(DEV),
                   b_s[:, :2].contiguous().to(DEV), out_dtype=torch.float32)                      # ragged K: silent


@pytest.mark.parametrize("M,N,K", [(7, 5, 100), (33, 130, 200), (3, 3, 1), (64, 64, 130)])
def test_gemm_ragged_k_scalar_path(M, N, K):
    """K not a multiple of 128: the tail block is shorter (masked loads at offical_kernel.py:82-83)."""
    g = torch.Generator().manual_seed(K)
    a = torch.randint(0, 0x70, (M, K), generator=g, dtype=torch.uint8).view(FP8)
    b = torch.randint(0, 0x70, (N, K), generator=g, dtype=torch.uint8).view(FP8)
    KB = (K + 127) // 128
    a_s = torch.rand(M, KB, generator=g) * 1e-2
    b_s = torch.rand((N + 127) // 128, KB, generator=g) * 1e-2
    ref = O.fp8_gemm(a, a_s, b, b_s, dtype=torch.float32)
    got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32)
    assert torch.allclose(got.cpu(), ref, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("M,N,K", [(256, 512, 1000), (16, 4096, 300), (1000, 260, 7170)])
def test_gemm_ragged_k_large_shapes_run_padded(M, N, K):
    """A larger problem with K % 128 != 0 is completed with zero columns and runs on the MFMA kernels: exact on
    integer operands, and equal to the scalar kernel's masked tail within fp32 summation order."""
    g = torch.Generator().manual_seed(K)
    ai = torch.randint(-4, 5, (M, K), generator=g)
    bi = torch.randint(-4, 5, (N, K), generator=g)
    KB, NB = (K + 127) // 128, (N + 127) // 128
    ae = torch.randint(-2, 3, (M, KB), generator=g)
    be = torch.randint(-2, 3, (NB, KB), generator=g)
    c = torch.zeros(M, N, dtype=torch.float64)
    for kb in range(KB):
        part = ai[:, kb * 128:(kb + 1) * 128].double() @ bi[:, kb * 128:(kb + 1) * 128].double().t()
        c += part * torch.exp2((ae[:, kb][:, None] + be[torch.arange(N) // 128, kb][None, :]).double())
    a, b = ai.float().to(FP8).to(DEV), bi.float().to(FP8).to(DEV)
    a_s, b_s = torch.exp2(ae.float()).to(DEV), torch.exp2(be.float()).to(DEV)
    got = m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.float32)
    assert torch.equal(got.cpu().double(), c)
    lib = _lib.load()
    ref = torch.full((M, N), float("nan"), device=DEV)
    assert lib.mdy_fp8_gemm_nt(a.data_ptr(), a_s.data_ptr(), KB, 1, b.data_ptr(), b_s.data_ptr(), ref.data_ptr(), None, M, N, K, 1,
                               None) == 0                       # the C entry point itself: scalar kernel, masked tail
    torch.cuda.synchronize()
    assert torch.equal(ref.cpu().double(), c)


def test_gemm_leading_dims_default_dtype_and_bias():
    a, a_s, wq, ws = quantized_problem("normal", 96, 384, 256, 5)
    a3, a3_s = a.reshape(2, 48, 256), a_s.reshape(2, 48, 2)
    got = m.fp8_gemm(a3.to(DEV), a3_s.to(DEV), wq.to(DEV), ws.to(DEV))
    assert got.shape == (2, 48, 384) and got.dtype == torch.get_default_dtype()
    ref = O.fp8_gemm(a3, a3_s, wq, ws, dtype=torch.float32)
    # fp32 output: the only differences left are summation order and the matrix core's
    # internal alignment of the 128 products of a K block
    assert torch.allclose(got.cpu(), ref, rtol=2e-3, atol=1e-3)
    bias = torch.randn(384).bfloat16()
    gb = m.fp8_gemm(a.to(DEV), a_s.to(DEV), wq.to(DEV), ws.to(DEV), out_dtype=torch.bfloat16, bias=bias.to(DEV))
    rb = O.fp8_gemm(a, a_s, wq, ws, dtype=torch.bfloat16, bias=bias)
    assert close(gb, rb)


# ------------------------------------------------------------------ DeepLinear path
@pytest.mark.parametrize("M,N,K", [(128, 1024, 1024), (64, 2048, 7168), (4, 128, 256), (4096, 1536, 7168)])
def test_fp8_matmul_column_major_scales(M, N, K):
    x = P.activations("normal", M, K, 3)
    w, _, _ = P.weights(N, K, 4)
    qa, sa, _, _ = m.quant_input(x.to(DEV), True)
    qb, sb, _, _ = m.quant_weight(w.to(DEV), True)
    assert sa.stride() == (1, qa.size(0))
    out = m.fp8_matmul(qa, sa, qb, sb)
    ra, rsa, _, _ = O.quant_input(x, True)
    rb, rsb, _, _ = O.quant_weight(w, True)
    rows = torch.unique(torch.cat([torch.arange(0, M, 37), torch.tensor([M - 1])]))
    ref = O.fp8_matmul(ra[rows].contiguous(), rsa[rows].contiguous(), rb, rsb)
    assert out.dtype == torch.bfloat16 and out.shape == (qa.size(0), qb.size(0))
    assert close(out[rows.to(DEV)], ref)
    buf = torch.empty_like(out)
    assert m.fp8_matmul(qa, sa, qb, sb, out=buf).data_ptr() == buf.data_ptr() and torch.equal(buf, out)


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape,N", [((2, 64, 512), 256), ((8, 1024), 384), ((1, 4, 7168), 2048)])
def test_deep_linear_forward(shape, N, bias):
    g = torch.Generator().manual_seed(sum(shape) + N)
    K = shape[-1]
    lin = m.DeepLinear(K, N, bias=bias, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(N, K, generator=g) * 0.02).bfloat16())
        if bias:
            lin.bias.copy_(torch.randn(N, generator=g).bfloat16())
    x = torch.randn(*shape, generator=g).bfloat16()
    ref = O.deep_linear_forward(x, lin.weight.detach(), lin.bias.detach() if bias else None)
    lin = lin.to(DEV)
    assert lin.cache_weight is False         # the reference re-quantizes on every call (fp8.py:320)
    with torch.no_grad():
        out_nocache = lin(x.to(DEV))
        assert getattr(lin, "_wq_cache", None) is None
        lin.cache_weight = True
        out = lin(x.to(DEV))
        cached = lin._wq_cache[1][0].data_ptr()
        out_again = lin(x.to(DEV))          # second call uses the cached quantized weight
        assert lin._wq_cache[1][0].data_ptr() == cached
        lin.fuse_bias = True
        out_fused = lin(x.to(DEV))
    assert out.shape == (*shape[:-1], N) and out.dtype == torch.bfloat16
    assert close_biased(out, ref, lin.bias.detach() if bias else None)
    assert torch.equal(out, out_again) and torch.equal(out, out_nocache)
    assert close_biased(out_fused, ref, lin.bias.detach() if bias else None)
    # sanity band against the unquantized layer (the reference prints ~0.017 mean abs error at d=4096)
    full = torch.nn.functional.linear(x.float(), lin.weight.detach().float().cpu(),
                                      lin.bias.detach().float().cpu() if bias else None)
    assert (out.float().cpu() - full).abs().mean() < 0.05


def test_deep_linear_cache_follows_weight_updates():
    lin = m.DeepLinear(256, 128, bias=False, dtype=torch.bfloat16, device=DEV)
    lin.cache_weight = True
    x = torch.randn(8, 256, device=DEV).bfloat16()
    with torch.no_grad():
        y0 = lin(x)
        lin.weight.mul_(2)                  # bumps the version counter: noticed without a call
        y1 = lin(x)
    assert torch.allclose(y1.float(), 2 * y0.float(), rtol=2e-2, atol=1e-3) and not torch.equal(y0, y1)


def test_deep_linear_cache_and_data_updates():
    """An update through `.data` (what Megatron's / apex's / DeepSpeed's optimizers do) bumps no version
    counter.  Without the cache (the default, as in the reference) the next forward sees it; with the cache it is
    seen after invalidate_weight_cache() / set_first_micro_batch(True), and the checking mode raises instead of
    multiplying by the stale copy."""
    x = torch.randn(8, 256, device=DEV).bfloat16()
    lin = m.DeepLinear(256, 128, bias=False, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        y0 = lin(x)
        v = lin.weight._version
        lin.weight.data.mul_(2)
        assert lin.weight._version == v      # the premise: nothing to observe
        y1 = lin(x)
    assert torch.allclose(y1.float(), 2 * y0.float(), rtol=2e-2, atol=1e-3) and not torch.equal(y0, y1)

    lin.cache_weight = True
    with torch.no_grad():
        y1c = lin(x)
        lin.weight.data.mul_(0.5)
        stale = lin(x)                       # documented: the cached copy is still the old weight
        assert torch.equal(stale, y1c)
        lin.invalidate_weight_cache()
        fresh = lin(x)
        assert torch.equal(fresh, y0)
        lin.weight.data.copy_(lin.weight.data * 2)
        lin.set_first_micro_batch(True)      # the reference's name for the same signal (manger.py:77-86)
        assert torch.equal(lin(x), y1)
        lin.set_first_micro_batch(False)     # later micro-batches: keep the copy
        ptr = lin._wq_cache[1][0].data_ptr()
        lin(x)
        assert lin._wq_cache[1][0].data_ptr() == ptr

    lin.check_weight_cache = True
    lin.invalidate_weight_cache()
    with torch.no_grad():
        lin(x)
        lin(x)                               # unchanged weight: the check passes
        lin.weight.data.mul_(2)
        with pytest.raises(RuntimeError, match="invalidate_weight_cache"):
            lin(x)
        lin.invalidate_weight_cache()
        assert torch.equal(lin(x), lin(x))


def test_fp8_mlp_sees_data_updates_after_invalidation():
    mlp = m.Fp8MLP(256, 256, device=DEV, dialect="deeplinear", fp8_dtype=torch.float8_e4m3fn)
    mlp.up_gate_proj.cache_weight = mlp.down_proj.cache_weight = True
    x = torch.randn(16, 256, device=DEV).bfloat16()
    with torch.no_grad():
        y0 = mlp(x)
        mlp.down_proj.weight.data.mul_(2)
        assert torch.equal(mlp(x), y0)
        mlp.down_proj.invalidate_weight_cache()
        y1 = mlp(x)
    assert torch.allclose(y1.float(), 2 * y0.float(), rtol=2e-2, atol=1e-3) and not torch.equal(y0, y1)


# ------------------------------------------------------------------ DeepLinear backward
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape,N", [((2, 128, 256), 256), ((512, 1024), 768), ((3, 50, 300), 200), ((1024, 7168), 1536)])
def test_deep_linear_backward(shape, N, bias):
    g = torch.Generator().manual_seed(sum(shape) + N + 1)
    K = shape[-1]
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    b = torch.randn(N, generator=g).bfloat16() if bias else None
    x = torch.randn(*shape, generator=g).bfloat16()
    dy = torch.randn(*shape[:-1], N, generator=g).bfloat16()
    ref_out = O.deep_linear_forward(x, w, b)
    ref_dx, ref_dw, ref_db = O.deep_linear_backward(x, w, dy, bias)

    lin = m.DeepLinear(K, N, bias=bias, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
        if bias:
            lin.bias.copy_(b)
    lin = lin.to(DEV)
    for cache in (True, False):
        lin.cache_weight = cache
        lin.zero_grad()
        xg = x.to(DEV).requires_grad_(True)
        out = lin(xg)
        out.backward(dy.to(DEV))
        assert close_biased(out, ref_out, b)
        assert xg.grad.shape == x.shape and xg.grad.dtype == torch.bfloat16
        assert lin.weight.grad.shape == (N, K) and lin.weight.grad.dtype == torch.bfloat16
        assert close(xg.grad, ref_dx)
        assert close(lin.weight.grad, ref_dw)
        if bias:
            assert torch.allclose(lin.bias.grad.float().cpu(), ref_db.float(), rtol=1e-2, atol=1e-2)
    # sanity band against the unquantized gradients
    xf, dyf = x.float().reshape(-1, K), dy.float().reshape(-1, N)
    dref, wref = (dyf @ w.float()).reshape(x.shape), dyf.t() @ xf
    assert (xg.grad.float().cpu() - dref).abs().mean() < 0.06 * dref.abs().mean()
    assert (lin.weight.grad.float().cpu() - wref).abs().mean() < 0.06 * wref.abs().mean()


def test_deep_linear_backward_partial_requirements():
    lin = m.DeepLinear(256, 256, bias=True, dtype=torch.bfloat16, device=DEV)
    x = torch.randn(64, 256, device=DEV).bfloat16()
    out = lin(x)                                  # input needs no gradient: only wgrad and grad_bias
    out.sum().backward()                          # the incoming gradient is an expanded (stride-0) tensor
    assert lin.weight.grad is not None and lin.bias.grad is not None
    ref = O.deep_linear_backward(x.cpu(), lin.weight.detach().cpu(), torch.ones(64, 256).bfloat16())
    assert close(lin.weight.grad, ref[1])
    lin.weight.requires_grad_(False); lin.bias.requires_grad_(False)
    xg = x.clone().requires_grad_(True)
    lin(xg).sum().backward()                      # only dgrad
    assert close(xg.grad, ref[0])


# ------------------------------------------------------------------ non-finite values
@pytest.mark.parametrize("M,N,K", [(256, 384, 512),       # MFMA tiles
                                   (8, 256, 512),         # weight-streaming kernel
                                   (130, 1100, 4224),     # split along K
                                   (16, 25600, 256),      # strip kernel
                                   (40, 48, 100)])        # one thread per element
def test_gemm_non_finite_values_follow_the_block_formula(M, N, K):
    """A NaN operand byte poisons exactly its output row / column, an infinite scale makes its row infinite
    with the sign of the block's partial sum: the same pattern as the reference's accumulation
    (offical_kernel.py:80-91) evaluated block by block on the CPU, in every kernel."""
    g = torch.Generator().manual_seed(M * 7 + N)
    a = torch.randint(-6, 7, (M, K), generator=g).float().to(FP8)
    b = torch.randint(-6, 7, (N, K), generator=g).float().to(FP8)
    KB, NB = (K + 127) // 128, (N + 127) // 128
    a_s = torch.rand(M, KB, generator=g) + 0.5
    b_s = torch.rand(NB, KB, generator=g) + 0.5
    au, bu = a.view(torch.uint8), b.view(torch.uint8)
    au[1, 3] = 0x7F                                     # NaN in activation row 1
    bu[5, K - 1] = 0xFF                                 # NaN in weight row 5 (last K element)
    a_s[2, KB - 1] = float("inf")                       # row 2: +-inf, or NaN where the block's partial sum is 0
    a_s[3, 0] = 0.0                                     # a zero scale drops the block
    ref = O.fp8_gemm_blockwise(a, a_s, b, b_s, dtype=torch.float32)
    got = m.fp8_gemm(a.to(DEV), a_s.to(DEV), b.to(DEV), b_s.to(DEV), out_dtype=torch.float32).cpu()
    assert torch.equal(torch.isnan(got), torch.isnan(ref))
    assert torch.isnan(got[1]).all() and torch.isnan(got[:, 5]).all()
    assert torch.equal(torch.isinf(got), torch.isinf(ref)) and torch.equal(got[torch.isinf(ref)], ref[torch.isinf(ref)])
    fin = torch.isfinite(ref)
    # fp32 sums of ~1e3-sized terms in a different order (and scale products rounded differently): a few ulps of 1e3
    assert fin[4:].any() and torch.allclose(got[fin], ref[fin], rtol=1e-4, atol=1e-2)
