"""CPU oracle for the block-wise FP8 linear path.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only `tests/`, `__graft_entry__.smoke()`
and the `cpu_baseline` leg of `bench.py` may import this module; the product
package (`mdy_triton_amd`) never imports anything from `oracle/` and has no CPU
fallback.

Every function restates, with torch CPU tensor ops in IEEE fp32, the algorithm
of one reference function and cites it.  All paths are under /root/reference.

Pinning status (what fixes each function besides its own formula):
  act_quant / quant_input / quant_weight / weight_quant_block
      the fp32->e4m3fn cast is pinned against the from-definition codec in
      oracle/fp8_format.py on every code, every rounding midpoint +-1 ulp,
      subnormals, 448/464/465, +-0, NaN, inf; the scale against numpy float32
      division; invariants (the amax element encodes to +-448, half-ulp
      reconstruction bound, idempotence) and hand-computed fixtures in
      tests/golden/.
  weight_dequant
      s == 1 reduces to the 256-entry decode table; one fp32 multiply + RNE
      to bf16 re-derived in numpy integer arithmetic.
  fp8_gemm
      float64 matmul on small shapes; exactly-representable integer cases that
      must match bit for bit; one-hot rows; single-scale-block perturbation.
  quant_grad_output / quant_input(only_forward=False) / per_token_cast_to_fp8 /
  group_per_token_cast_to_fp8 / per_block_cast_to_fp8
      reduce to the pinned forward quantizers: row-wise copy == quant_input, the
      column-wise transposed copy == quant_input of the transposed matrix, the
      block-scaled transposed copy == quant_weight's; padding, strides and single
      tiles re-derived by brute force in numpy (tests/test_oracle.py).
  silu_fwd / silu_bwd / silu_act_quant
      floating point: compared with torch.nn.functional.silu and its autograd
      gradient (library routines) and closed forms; the quantizer half is act_quant.
  deep_linear_backward / fp8_grouped_matmul
      compositions of the above (per group: fp8_gemm); checked against unquantized
      fp32 gradients within the quantization error band and for operand roles
      (swapping x and dy transposes wgrad).
  act_quant_block / fp8_matmul_official / fp8_linear_forward / fp8_linear_backward  (the reference's Fp8Linear)
      act_quant_block(x) is act_quant; act_quant_block(x, transpose=True) must equal act_quant of the zero-padded
      transposed matrix (checked, with a brute-force group loop on top); the GEMM with row scales on both operands
      against a float64 evaluation of its formula, exactly-representable integer cases, and its reduction to the
      pinned fp8_gemm when the weight-row scales are constant within each 128-row block.
  fp8_padding / fp8_unpadding
      pure row moves: brute-force row-by-row loops on small inputs, the round trip
      unpad(pad(x)) == x, zero padding rows, slot starts at multiples of 256.
  fp8_matmul (DeepLinear's GEMM)
      PARITY UNPINNED at the third-party boundary: the reference calls
      `deep_gemm.gemm_fp8_fp8_bf16_nt` (dpsk_fp8linear/fp8.py:310; the grouped
      call is megatron_patchs/fp8_matmul.py:412), an
      un-vendored, un-pinned package whose source is not in the reference and
      whose only recorded outputs are unseeded notebook prints.  The oracle
      follows the in-tree formula with the same contract
      (deepseekv3/offical_kernel.py:81-92) instead.
"""
from typing import Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0
BLOCK = 128


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# ----------------------------------------------------------------------------
# DeepSeek "official" dialect
# ----------------------------------------------------------------------------
def act_quant(x: torch.Tensor, block_size: int = BLOCK) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per 128 contiguous elements: s = max|x| / 448 ; y = (x / s) -> e4m3fn.

    Follows triton_kernels/deepseekv3/offical_kernel.py:9-18 (kernel) and
    :21-28 (launcher: contiguous, last dim % block_size == 0, y same shape,
    s shape [..., K/block_size] fp32).  No eps, no clamp: an all-zero group gives
    s = 0 and y = 0/0 = NaN.
    """
    assert x.is_contiguous()
    assert x.size(-1) % block_size == 0
    xf = x.detach().cpu().float().reshape(-1, block_size)
    s = xf.abs().amax(dim=-1) / FP8_MAX                     # offical_kernel.py:14
    y = (xf / s[:, None]).to(FP8)                           # offical_kernel.py:15-16
    y = y.reshape(x.shape)
    s = s.reshape(*x.shape[:-1], x.size(-1) // block_size)
    return y, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = BLOCK,
                   dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y[m, n] = fp32(x[m, n]) * s[m // 128, n // 128], rounded once to `dtype`.

    Follows offical_kernel.py:31-43 (kernel; edge tiles masked at :39) and :46-53
    (2-D contiguous inputs; output dtype is the caller's default dtype at :50).
    """
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    M, N = x.shape
    assert s.shape == (_cdiv(M, block_size), _cdiv(N, block_size))
    xf = x.detach().cpu().float()
    sf = s.detach().cpu().float()
    sfull = sf.repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (xf * sfull).to(dtype)                           # offical_kernel.py:42


def dequant_rows(a: torch.Tensor, a_s: torch.Tensor, block_size: int = BLOCK) -> torch.Tensor:
    """fp32 a[m, k] * a_s[m, k // 128] (activation side of the GEMM)."""
    K = a.size(-1)
    af = a.detach().cpu().float().reshape(-1, K)
    sf = a_s.detach().cpu().float().reshape(af.size(0), -1)
    return af * sf.repeat_interleave(block_size, 1)[:, :K]


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor,
             dtype: torch.dtype = torch.bfloat16, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C = A . B^T with per-128-K scales: dequantize both operands, fp32 matmul.

    C[m, n] = sum_kb (sum_{k in kb} a[m,k] b[n,k]) * a_s[m,kb] * b_s[n//128,kb]
    (offical_kernel.py:81-92; launcher :100-109: a [.., K], b [N, K], a_s
    [.., cdiv(K,128)], b_s [cdiv(N,128), cdiv(K,128)], out [.., N]).  Equal in
    exact arithmetic to dequant(a) @ dequant(b).T, which is what is evaluated
    here in fp32 and what the parity tolerance (rtol 1e-2, atol 1e-2) refers to.
    """
    K = a.size(-1)
    N = b.size(0)
    ad = dequant_rows(a, a_s)
    bd = weight_dequant(b.reshape(N, K).contiguous(), b_s.contiguous(), dtype=torch.float32)
    c = ad @ bd.t()
    if bias is not None:
        c = c + bias.detach().cpu().float()
    return c.to(dtype).reshape(*a.shape[:-1], N)


def fp8_gemm_f64(a, a_s, b, b_s) -> torch.Tensor:
    """Same contraction in float64 (tight truth for small shapes); returns float64 [M, N]."""
    K = a.size(-1)
    N = b.size(0)
    ad = a.detach().cpu().double().reshape(-1, K) * \
        a_s.detach().cpu().double().reshape(-1, a_s.size(-1)).repeat_interleave(BLOCK, 1)[:, :K]
    bd = b.detach().cpu().double().reshape(N, K) * \
        b_s.detach().cpu().double().repeat_interleave(BLOCK, 0)[:N].repeat_interleave(BLOCK, 1)[:, :K]
    return ad @ bd.t()


def fp8_gemm_blockwise(a, a_s, b, b_s, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The accumulation order of the kernel itself: one fp32 partial dot per
    128-K block, scaled, then added (offical_kernel.py:80-91).  Small shapes only."""
    K = a.size(-1)
    N = b.size(0)
    af = a.detach().cpu().float().reshape(-1, K)
    bf = b.detach().cpu().float().reshape(N, K)
    M = af.size(0)
    asf = a_s.detach().cpu().float().reshape(M, -1)
    bsf = b_s.detach().cpu().float()
    acc = torch.zeros(M, N, dtype=torch.float32)
    nrow = torch.arange(N) // BLOCK
    for kb in range(_cdiv(K, BLOCK)):
        k0, k1 = kb * BLOCK, min(K, (kb + 1) * BLOCK)
        part = af[:, k0:k1] @ bf[:, k0:k1].t()
        acc += part * asf[:, kb][:, None] * bsf[nrow, kb][None, :]
    return acc.to(dtype).reshape(*a.shape[:-1], N)


def weight_quant_block(w: torch.Tensor, block_size: int = BLOCK, dtype: torch.dtype = FP8) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 block quantizer without eps: s = max|blk| / MAX ; y = blk / s.

    Follows triton_kernels/deepseekv3/fp8_kernel.py:117-122 with
    MAX = finfo(dtype).max (:133: 448 for e4m3fn, 57344 for the reference's default e5m2); this is how
    block-quantized test weights are produced.  Requires both dims % 128 == 0 (U = M // BLOCK_M at :128-129).
    """
    N, K = w.shape
    assert N % block_size == 0 and K % block_size == 0
    wf = w.detach().cpu().float().reshape(N // block_size, block_size, K // block_size, block_size)
    s = wf.abs().amax(dim=(1, 3)) / torch.finfo(dtype).max
    y = (wf / s[:, None, :, None]).to(dtype).reshape(N, K)
    return y, s


# ----------------------------------------------------------------------------
# DeepLinear dialect (clamp + eps, padded, column-major activation scales)
# ----------------------------------------------------------------------------
def _scale_from_amax(amax: torch.Tensor) -> torch.Tensor:
    """clamp(amax, 0, 1e4) + 1e-8, then / 448, all in fp32 (fp8.py:109-110, 194-195)."""
    return (amax.clamp(min=0.0, max=1e4) + torch.tensor(1e-8, dtype=torch.float32)) / 448


def _cast_sat(v: torch.Tensor) -> torch.Tensor:
    """fp32 -> e4m3fn with finite overflow saturating at +-448.

    The reference's cast is the implicit one of `tl.store` to an fp8 pointer
    (fp8.py:112, 198), which is `cvt.rn.satfinite` on the hardware it targets;
    torch's CPU cast alone would turn |v| >= 465 into NaN.
    """
    return torch.where(v.isnan(), v, v.clamp(-FP8_MAX, FP8_MAX)).to(FP8)


def quant_input(x: torch.Tensor, only_forward: bool = True):
    """1x128 activation quantizer of DeepLinear.

    Follows dpsk_fp8linear/fp8.py:87-120 (kernel) and :122-161 (launcher):
    PN = cdiv(K,256)*256; PM = cdiv(M,4)*4 (forward only) or cdiv(M,256)*256;
    padded elements read as 0 (:108); y [PM, PN] row-major; scales written
    S[kb*PM + m] (:113) and returned transposed: logical [PM, B], strides (1, PM).
    With only_forward=False also the transposed copy quantized per 128x128 block
    with the block's max of the row amax' values (:115-120): y_t [PN, PM],
    s_t [B, A] with A = PM/128.
    """
    M, K = x.shape
    PN = _cdiv(K, 256) * 256
    B = PN // BLOCK
    PM = _cdiv(M, 4) * 4 if only_forward else _cdiv(M, 256) * 256
    xp = torch.zeros(PM, PN, dtype=torch.float32)
    xp[:M, :K] = x.detach().cpu().float()
    g = xp.reshape(PM, B, BLOCK)
    amaxp = g.abs().amax(-1).clamp(min=0.0, max=1e4) + torch.tensor(1e-8, dtype=torch.float32)
    scale = amaxp / 448                                      # [PM, B]
    y = _cast_sat(g / scale[:, :, None]).reshape(PM, PN)
    s = scale.t().contiguous().t()                           # logical [PM, B], strides (1, PM)
    if only_forward:
        return y, s, None, None
    A = PM // BLOCK
    blk_amax = amaxp.reshape(A, BLOCK, B).amax(1)            # fp8.py:116 max over rows of the tile
    blk_scale = blk_amax / 448                               # [A, B]
    yb = g.reshape(A, BLOCK, B, BLOCK) / blk_scale[:, None, :, None]
    y_t = _cast_sat(yb).reshape(PM, PN).t().contiguous()     # [PN, PM]
    s_t = blk_scale.t().contiguous()                         # [B, A] (fp8.py:120)
    return y, s, y_t, s_t


def quant_weight(w: torch.Tensor, only_forward: bool = True):
    """128x128 weight quantizer of DeepLinear.

    Follows fp8.py:171-203 (kernel) and :206-247 (launcher): rows padded to 128
    (256 when training), columns to 256; y [PM, PN]; s [A, B] row-major (:199);
    with only_forward=False also y_t [PN, PM] and s_t [B, A] (:201-203).
    """
    N, K = w.shape
    BA = 128 if only_forward else 256
    PM, PN = _cdiv(N, BA) * BA, _cdiv(K, 256) * 256
    A, B = PM // BLOCK, PN // BLOCK
    wp = torch.zeros(PM, PN, dtype=torch.float32)
    wp[:N, :K] = w.detach().cpu().float()
    g = wp.reshape(A, BLOCK, B, BLOCK)
    scale = _scale_from_amax(g.abs().amax(dim=(1, 3)))       # [A, B]
    y = _cast_sat(g / scale[:, None, :, None]).reshape(PM, PN)
    if only_forward:
        return y, scale, None, None
    return y, scale, y.t().contiguous(), scale.t().contiguous()


def quant_grad_output(dy: torch.Tensor):
    """Row-wise 1x128 and column-wise 128x1 quantization of the output gradient.

    Follows fp8.py:13-44 (kernel) and :47-77 (launcher): PM, PN padded to 256;
    y [PM, PN] with scales returned as logical [PM, B] (col-major); y_t [PN, PM]
    quantized along M in groups of 128 with scales returned as logical [PN, A].
    """
    M, N = dy.shape
    PM, PN = _cdiv(M, 256) * 256, _cdiv(N, 256) * 256
    A, B = PM // BLOCK, PN // BLOCK
    xp = torch.zeros(PM, PN, dtype=torch.float32)
    xp[:M, :N] = dy.detach().cpu().float()
    g = xp.reshape(PM, B, BLOCK)
    scale = _scale_from_amax(g.abs().amax(-1))               # [PM, B]
    y = _cast_sat(g / scale[:, :, None]).reshape(PM, PN)
    s = scale.t().contiguous().t()
    gt = xp.t().contiguous().reshape(PN, A, BLOCK)
    scale_t = _scale_from_amax(gt.abs().amax(-1))            # [PN, A]
    y_t = _cast_sat(gt / scale_t[:, :, None]).reshape(PN, PM)
    s_t = scale_t.t().contiguous().t()
    return y, s, y_t, s_t


def add_bias(x: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """x[r, :] = (fp32(x[r, :]) + fp32(b)) -> x.dtype  (fp8.py:283-295, 297-305)."""
    return (x.detach().cpu().float() + b.detach().cpu().float()).to(x.dtype)


def add_grad(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """x = (fp32(x) + fp32(y)) -> x.dtype  (megatron_patchs/add_kernel.py:41-62)."""
    return (x.detach().cpu().float() + y.detach().cpu().float()).to(x.dtype)


def fp8_matmul(qa, sa, qb, sb) -> torch.Tensor:
    """bf16 out[PM, PNw] of DeepLinear's GEMM call (fp8.py:307-311); sa may be
    column-major.  Third-party boundary: see the module header."""
    return fp8_gemm(qa, sa.contiguous(), qb, sb.contiguous(), dtype=torch.bfloat16)


def deep_linear_forward(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """Composition of fp8.py:313-328: flatten, quant_input, quant_weight,
    fp8_matmul, add_bias, view back.  Rows and columns the quantizers added as
    padding are dropped before the bias (the reference's own view only works
    when there are none: M % 4 == 0 and N % 128 == 0)."""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    qa, sa, _, _ = quant_input(x2, True)
    qb, sb, _, _ = quant_weight(weight, True)
    out = fp8_matmul(qa, sa, qb, sb)[:x2.size(0), :weight.size(0)].contiguous()
    if bias is not None:
        out = add_bias(out, bias)
    return out.view(*shape[:-1], -1)


def deep_linear_backward(x: torch.Tensor, weight: torch.Tensor, grad_output: torch.Tensor, has_bias: bool = True):
    """Composition of fp8.py:331-344 on the tensors the forward saved (:318-321):
    dgrad = fp8_matmul(q(dy), q_t(W)), wgrad = fp8_matmul(q_t(dy), q_t(x)), grad_bias = dy.sum(0).

    The reference multiplies the padded operands and views the result with the input's
    shape, which only works when no padding was added; here the padded rows and columns
    are dropped, which is the same thing for shapes that are multiples of 256.
    """
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    M, K = x2.shape
    N = weight.size(0)
    dy = grad_output.reshape(-1, N)
    _, _, q_inp_t, s_inp_t = quant_input(x2, False)
    _, _, q_w_t, s_w_t = quant_weight(weight, False)
    q_dy, s_dy, q_dy_t, s_dy_t = quant_grad_output(dy)
    dgrad = fp8_matmul(q_dy, s_dy, q_w_t, s_w_t)[:M, :K].reshape(shape)
    wgrad = fp8_matmul(q_dy_t, s_dy_t, q_inp_t, s_inp_t)[:N, :K]
    # torch's bf16 sum accumulates in fp32 and rounds once (fp8.py:343)
    grad_bias = dy.detach().cpu().float().sum(0).to(dy.dtype) if has_bias else None
    return dgrad, wgrad, grad_bias


# ----------------------------------------------------------------------------
# SwiGLU before the down projection (floating point: compared with a tolerance)
# ----------------------------------------------------------------------------
def _split_up_gate(x: torch.Tensor, order: str):
    assert order in ("up-gate", "gate-up")
    N = x.size(-1) // 2
    xf = x.detach().cpu().float()
    first, second = xf[..., :N], xf[..., N:]
    return (first, second) if order == "up-gate" else (second, first)     # fp8_kernel.py:327-332


def silu_fwd(x: torch.Tensor, order: str = "up-gate") -> torch.Tensor:
    """y = (gate * sigmoid(gate)) * up in fp32, rounded once to x.dtype (fp8_kernel.py:335-344)."""
    up, gate = _split_up_gate(x, order)
    return ((gate * torch.sigmoid(gate)) * up).to(x.dtype)


def silu_bwd(dy: torch.Tensor, x: torch.Tensor, order: str = "up-gate") -> torch.Tensor:
    """fp8_kernel.py:369-382: dup = act*dy, dgate = (sig + act*(1-sig)) * (up*dy), each rounded to dy.dtype."""
    up, gate = _split_up_gate(x, order)
    d = dy.detach().cpu().float().reshape(up.shape)
    sig = torch.sigmoid(gate)
    act = sig * gate
    dup = (act * d).to(dy.dtype)
    dgate = ((sig + act * (1 - sig)) * (up * d)).to(dy.dtype)
    return torch.cat([dup, dgate] if order == "up-gate" else [dgate, dup], dim=-1)


def silu_act_quant(x: torch.Tensor, order: str = "up-gate"):
    """The unfused pair of the FP8 MLP (fp8_kernel.py:447-450): act = silu_fwd(x); act_quant(act)."""
    act = silu_fwd(x, order)
    y, s = act_quant(act.contiguous())
    return y, s, act


# ----------------------------------------------------------------------------
# Grouped (mixture-of-experts) operators of megatron_patchs/fp8_matmul.py
# ----------------------------------------------------------------------------
def per_token_cast_to_fp8(x: torch.Tensor, output_transpose: bool = False):
    """fp8_matmul.py:96-135: quant_input's arithmetic; with output_transpose rows pad to 128 (not 256)
    and the transposed copy is quantized column-wise in groups of 128 rows."""
    if not output_transpose:
        return quant_input(x, True)
    M, N = x.shape
    PM, PN = _cdiv(M, 128) * 128, _cdiv(N, 256) * 256
    xp = torch.zeros(PM, PN, dtype=torch.float32)
    xp[:M, :N] = x.detach().cpu().float()
    g = xp.reshape(PM, PN // BLOCK, BLOCK)
    scale = _scale_from_amax(g.abs().amax(-1))
    y = _cast_sat(g / scale[:, :, None]).reshape(PM, PN)
    gt = xp.t().contiguous().reshape(PN, PM // BLOCK, BLOCK)
    scale_t = _scale_from_amax(gt.abs().amax(-1))
    y_t = _cast_sat(gt / scale_t[:, :, None]).reshape(PN, PM)
    return y, scale.t().contiguous().t(), y_t, scale_t.t().contiguous().t()


def group_per_token_cast_to_fp8(x_all: torch.Tensor, m_splits):
    """fp8_matmul.py:218-247: rows quantized over the whole matrix (scales [N/128, Mtot] returned
    transposed), and per group the column-wise quantized transpose."""
    Mtot, N = x_all.shape
    ys, ss, yts, sts = [], [], [], []
    for x in x_all.split(list(m_splits), 0):
        assert x.size(0) % 256 == 0 and N % 256 == 0
        if x.size(0) == 0:
            yts.append(torch.empty(N, 0, dtype=FP8)); sts.append(torch.empty(0, N).t()); continue
        y, s, y_t, s_t = per_token_cast_to_fp8(x, True)
        ys.append(y); ss.append(s.contiguous()); yts.append(y_t); sts.append(s_t)
    y_all = torch.cat(ys, 0)
    s_all = torch.cat(ss, 0).t().contiguous().t()
    return y_all, s_all, yts, sts


def per_block_cast_to_fp8(ws, output_normal: bool = True, output_transpose: bool = False):
    """fp8_matmul.py:334-392 for a list of equally shaped weights (stacked along a leading dimension)."""
    ws = list(ws) if isinstance(ws, (list, tuple)) else [ws]
    M, N = ws[0].shape
    BA, BB = (256 if output_transpose else 128), (256 if output_normal else 128)
    PM, PN = _cdiv(M, BA) * BA, _cdiv(N, BB) * BB
    A, B = PM // BLOCK, PN // BLOCK
    ys, ss = [], []
    for w in ws:
        wp = torch.zeros(PM, PN, dtype=torch.float32)
        wp[:M, :N] = w.detach().cpu().float()
        g = wp.reshape(A, BLOCK, B, BLOCK)
        scale = _scale_from_amax(g.abs().amax(dim=(1, 3)))
        ys.append(_cast_sat(g / scale[:, None, :, None]).reshape(PM, PN)); ss.append(scale)
    y, s = torch.stack(ys), torch.stack(ss)
    post = (lambda t: t.squeeze(0)) if len(ws) == 1 else (lambda t: t)
    out = ()
    if output_normal:
        out += (post(y), post(s))
    if output_transpose:
        out += (post(y.transpose(1, 2).contiguous()), post(s.transpose(1, 2).contiguous()))
    return out


def fp8_grouped_matmul(qa, sa, qb, sb, m_splits, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8_matmul.py:400-413: row m of group g is multiplied with weight g (one fp8_gemm per group)."""
    outs, row = [], 0
    sa = sa.contiguous()
    for g, mg in enumerate(m_splits):
        outs.append(fp8_gemm(qa[row:row + mg], sa[row:row + mg], qb[g], sb[g], dtype=torch.bfloat16,
                             bias=None if bias is None else bias[g]) if mg > 0
                    else torch.empty(0, qb.size(1), dtype=torch.bfloat16))
        row += mg
    return torch.cat(outs, 0)


def fp8_padding(inp: torch.Tensor, m_splits, multiple: int = 256):
    """Fp8Padding (megatron_patchs/dpsk_grouped_linear.py:798-902): group g's m_splits[g] rows move to the start of a
    slot of cdiv(m, 256) * 256 rows, the rest of the slot is zero (TransformerEngine's multi_padding_fused, called at
    :817).  Returns (padded [sum pad(m), H], padded_m_splits)."""
    x = inp.detach().cpu().reshape(-1, inp.shape[-1])
    pads = [(int(m) + multiple - 1) // multiple * multiple for m in m_splits]
    out = torch.zeros(sum(pads), x.size(1), dtype=x.dtype)
    src = dst = 0
    for m, pm in zip(m_splits, pads):
        out[dst:dst + m] = x[src:src + m]
        src += m
        dst += pm
    return out, pads


def fp8_unpadding(inp: torch.Tensor, m_splits, multiple: int = 256) -> torch.Tensor:
    """Fp8Unpadding (dpsk_grouped_linear.py:690-793): torch.split by the padded sizes, the first m_splits[g] rows of
    every piece, torch.cat (:703-706)."""
    x = inp.detach().cpu().reshape(-1, inp.shape[-1])
    pads = [(int(m) + multiple - 1) // multiple * multiple for m in m_splits]
    pieces = torch.split(x, pads)
    return torch.cat([p[:m] for p, m in zip(pieces, m_splits)], 0)


# ---------------------------------------------------------------------------
# The official-dialect linear layer of deepseekv3/fp8_kernel.py (Fp8Linear)
# ---------------------------------------------------------------------------
def act_quant_block(x: torch.Tensor, transpose: bool = False, dtype: torch.dtype = FP8):
    """fp8_kernel.py:62-87 (kernel :14-60): s = max|group| / finfo(dtype).max over 128 consecutive elements of a row
    (MAX at :82; 448 for e4m3fn, 57344 for e5m2), y = x / s cast to dtype, no clamp, no eps.  transpose=True quantizes x^T (the flattened [M, N] input along M); a last
    group shorter than 128 is completed with zeros (the kernel's boundary_check / padding_option='zero', :47-50).
    Returns (y, s): y like x and s [..., N/128], or y [N, M] and s [N, cdiv(M, 128)]."""
    x2 = x.detach().cpu().float().reshape(-1, x.shape[-1])
    if transpose:
        x2 = x2.t()
    R, C = x2.shape
    PC = _cdiv(C, BLOCK) * BLOCK
    xp = torch.zeros(R, PC, dtype=torch.float32)
    xp[:, :C] = x2
    g = xp.reshape(R, PC // BLOCK, BLOCK)
    s = g.abs().amax(-1) / torch.finfo(dtype).max
    y = (g / s[:, :, None]).to(dtype).reshape(R, PC)[:, :C].contiguous()
    if transpose:
        return y, s
    return y.reshape(x.shape), s.reshape(*x.shape[:-1], PC // BLOCK)


def fp8_matmul_official(x, w, scale_x, scale_w, bias: Optional[torch.Tensor] = None, have_w: bool = True) -> torch.Tensor:
    """fp8_kernel.py:214-252.  have_w=True: the block-scaled GEMM of offical_kernel.py with the bias added in fp32
    before the bf16 cast (:207-209) - the weight scale of output column n is row n // 128 of scale_w (the kernel's
    `pid_n * stride_sw1` with 256-wide tiles addresses other rows; that indexing slip is not followed).  have_w=False:
    both operands carry one scale per row and 128 columns (:196-203): y = dequant(x) . dequant(w)^T."""
    if have_w:
        x2 = x.reshape(-1, x.shape[-1])
        return fp8_gemm(x2, scale_x.reshape(x2.size(0), -1), w, scale_w, dtype=torch.bfloat16, bias=bias).reshape(*x.shape[:-1], -1)
    assert bias is None

    def deq(q, s):
        q = q.detach().cpu().float()
        R, C = q.shape
        PC = _cdiv(C, BLOCK) * BLOCK
        qp = torch.zeros(R, PC)
        qp[:, :C] = q
        return (qp.reshape(R, PC // BLOCK, BLOCK) * s.detach().cpu().float().reshape(R, -1)[:, :, None]).reshape(R, PC)
    return (deq(x, scale_x) @ deq(w, scale_w).t()).to(torch.bfloat16)


def fp8_linear_forward(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], dtype: torch.dtype = FP8) -> torch.Tensor:
    """_Fp8LinearFunction.forward (fp8_kernel.py:261-272)."""
    x2 = x.detach().cpu().reshape(-1, x.shape[-1])
    qx, sx = act_quant_block(x2, dtype=dtype)
    qw, sw = weight_quant_block(w.detach().cpu(), dtype=dtype)
    return fp8_matmul_official(qx, qw, sx, sw, bias, True).reshape(*x.shape[:-1], -1)


def fp8_linear_backward(x: torch.Tensor, w: torch.Tensor, dy: torch.Tensor, has_bias: bool = True, dtype: torch.dtype = FP8):
    """_Fp8LinearFunction.backward (fp8_kernel.py:274-301): (dx, dw, dbias)."""
    x2 = x.detach().cpu().reshape(-1, x.shape[-1])
    dy2 = dy.detach().cpu().reshape(-1, dy.shape[-1])
    dbias = dy2.sum(0) if has_bias else None
    qxt, sxt = act_quant_block(x2, transpose=True, dtype=dtype)
    qdy, sdy = act_quant_block(dy2, dtype=dtype)
    qdyt, sdyt = act_quant_block(dy2, transpose=True, dtype=dtype)
    qwt, swt = weight_quant_block(w.detach().cpu().t().contiguous(), dtype=dtype)
    dx = fp8_matmul_official(qdy, qwt, sdy, swt, None, True)
    dw = fp8_matmul_official(qdyt, qxt, sdyt, sxt, None, False)
    return dx.reshape(x.shape), dw, dbias
