"""mdy_fp8_gemm_nt_static_ws: the workspace GEMM for callers that cannot allocate.  Called through the C ABI
and compared bit for bit with mdy_fp8_gemm_nt_ws (same kernels, the scratch memory being the library's static
device array instead of a caller's buffer), twice in a row, the second call with a smaller input, so that
whatever the first call left in the shared array must not leak into the second result."""
import numpy as np
import pytest
import torch

from mdy_triton_amd import _lib
from oracle import oracle as O
from tests import problems as P

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
DEV = "cuda:0"


def _problem(M, N, K, seed):
    x = P.activations("normal", M, K, seed)
    a, a_s = O.act_quant(x)
    _, wq, ws = P.weights(N, K, seed + 1000)
    return [t.to(DEV) for t in (a, a_s, wq, ws)]


def _call(entry, a, a_s, b, b_s, dtype, bias=None, ws=None):
    lib = _lib.load()
    M, K = a.shape
    N = b.shape[0]
    c = torch.full((M, N), float("nan"), device=DEV, dtype=dtype)
    code = 0 if dtype == torch.bfloat16 else 1
    head = (a.data_ptr(), a_s.data_ptr(), K // 128, 1, b.data_ptr(), b_s.data_ptr(), c.data_ptr(),
            bias.data_ptr() if bias is not None else None, M, N, K, code)
    if entry == "static":
        rc = lib.mdy_fp8_gemm_nt_static_ws(*head, None)
    else:
        rc = lib.mdy_fp8_gemm_nt_ws(*head, ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, None)
    torch.cuda.synchronize()
    return rc, c


def _bits(t):
    return t.cpu().view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32).numpy()


# (first call, second smaller call): split along K with 128x128 / 128x64 tiles and, for (40, 300, 8192), the whole-line kernel over
# slabs of K; then a shape that needs no scratch
CASES = [((256, 4096, 4096), (128, 1536, 4096)),
         ((130, 1100, 5120), (40, 300, 8192)),
         ((128, 2112, 7168), (16, 2048, 7168)),
         ((64, 2048, 7168), (33, 130, 4096))]


@pytest.mark.parametrize("first,second", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_workspace_matches_caller_workspace(first, second, dtype):
    lib = _lib.load()
    assert lib.mdy_fp8_gemm_static_workspace_bytes() == 32 << 20
    assert lib.mdy_fp8_gemm_static_workspace_init() == 0
    for i, (M, N, K) in enumerate((first, second)):
        a, a_s, b, b_s = _problem(M, N, K, 7 * M + N + i)
        bias = torch.randn(N, generator=torch.Generator().manual_seed(N)).bfloat16().to(DEV) if i == 0 else None
        need = lib.mdy_fp8_gemm_workspace_bytes(M, N, K)
        if i == 0:
            assert need > 0, "the first call of every case is meant to use the scratch memory"
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        rc_ws, want = _call("ws", a, a_s, b, b_s, dtype, bias, ws)
        rc_st, got = _call("static", a, a_s, b, b_s, dtype, bias)
        assert rc_ws == 0 and rc_st == 0, lib.mdy_fp8_last_error()
        assert np.array_equal(_bits(got), _bits(want))
        # and within the GEMM tolerance of the oracle (rtol = atol = 1e-2)
        ref = O.fp8_gemm(a.cpu(), a_s.cpu(), b.cpu(), b_s.cpu(), dtype=dtype).float()
        if bias is not None:
            ref = ref + bias.float().cpu()
        assert torch.allclose(got.float().cpu(), ref, rtol=1e-2, atol=2e-2 if bias is not None else 1e-2)


def test_static_workspace_rejects_what_does_not_fit():
    """A shape whose scratch need exceeds the static array is refused before any launch; argument errors are
    reported as by the workspace entry point."""
    lib = _lib.load()
    limit = lib.mdy_fp8_gemm_static_workspace_bytes()
    # the transposed-scale copy of this shape alone is 2^20 rows x 128 K blocks x 4 bytes = 512 MiB, whatever the CU count
    M, N, K = 1 << 20, 256, 16384
    assert lib.mdy_fp8_gemm_workspace_bytes(M, N, K) > limit
    one = torch.zeros(16, dtype=torch.uint8, device=DEV)
    # pointers are never dereferenced: the call is rejected on the sizes alone
    rc = lib.mdy_fp8_gemm_nt_static_ws(one.data_ptr(), one.data_ptr(), K // 128, 1, one.data_ptr(), one.data_ptr(),
                                       one.data_ptr(), None, M, N, K, 0, None)
    assert rc == -2 and b"static buffer" in lib.mdy_fp8_last_error()
    assert lib.mdy_fp8_gemm_nt_static_ws(None, one.data_ptr(), 1, 1, one.data_ptr(), one.data_ptr(), one.data_ptr(), None,
                                         4, 4, 128, 0, None) == -1
    assert lib.mdy_fp8_gemm_nt_static_ws(one.data_ptr(), one.data_ptr(), 1, 1, one.data_ptr(), one.data_ptr(),
                                         one.data_ptr(), None, 4, 4, 128, 7, None) == -4
    assert lib.mdy_fp8_gemm_nt_static_ws(one.data_ptr(), one.data_ptr(), 1, 1, one.data_ptr(), one.data_ptr(),
                                         one.data_ptr(), None, 0, 4, 128, 0, None) == 0
