"""Seeded synthetic inputs of the benchmark configurations (generated on the CPU so
that the oracle and the device see identical bits)."""
import torch

from oracle import oracle as O


def activations(kind: str, M: int, K: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    if kind == "outliers":          # 1 % of the entries x10
        mask = torch.rand(M, K, generator=g) < 0.01
        x = torch.where(mask, x * 10, x)
    elif kind == "heavy":           # SiLU-gated look-alike: N(0,1) * |N(0,1)|
        x = x * torch.randn(M, K, generator=g).abs()
    elif kind != "normal":
        raise ValueError(kind)
    return x.bfloat16()


def weights_bf16(N: int, K: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(N, K, generator=g) * 0.02).bfloat16()


def weights(N: int, K: int, seed: int):
    """bf16 N(0, 0.02) weights, block-quantized 128x128 (rows padded for the quantizer
    only); returns (w_bf16 [N,K], wq e4m3fn [N,K], ws fp32 [ceil(N/128), K/128])."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    Np = (N + 127) // 128 * 128
    if Np != N:
        wp = torch.zeros(Np, K, dtype=torch.bfloat16)
        wp[:N] = w
        wq, ws = O.weight_quant_block(wp)
        wq = wq[:N].contiguous()
    else:
        wq, ws = O.weight_quant_block(w)
    return w, wq, ws


CONFIGS = {
    # name: (activation kind, M, N, K)
    "C1_cpu_reference": ("normal", 128, 1024, 1024),
    "C2_q_a_proj": ("outliers", 4096, 1536, 7168),
    "C3_mlp_up_gate": ("normal", 4096, 18432, 7168),
    "C4_mlp_down": ("heavy", 4096, 7168, 18432),
}
DECODE_SHAPES = [(M, N, K) for M in (1, 16, 64) for (N, K) in ((7168, 2048), (2048, 7168))]
