"""The operators under HIP graph capture: none of them allocates, synchronizes or reads back on its own
(the workspace of the K-split / scale-transposing GEMM paths comes from torch's allocator, which serves
captures from a private pool), so an inference step can be recorded once and replayed.  Every replay is
compared bit for bit with the eager result for the same input, with eager work and synchronizations of
the program's own between the replays."""
import pytest
import torch

import mdy_triton_amd as m

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bf16(rows, cols, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, cols, generator=g) * scale).bfloat16().to(DEV)


def mlp_step(x, lin_in, w_down_q, w_down_s):
    """up/gate projection (DeepLinear, cached weight) -> fused SwiGLU + quantizer -> down projection."""
    h = lin_in(x)
    q, s = m.silu_act_quant(h, "up-gate")
    return m.fp8_gemm(q, s, w_down_q, w_down_s)


# rows: decode (small-M kernel), K-split with workspace, tile kernels
@pytest.mark.parametrize("M", [4, 128, 1024])
def test_mlp_step_replays_bit_identically(M):
    K, F = 2048, 4096                      # model width, 2 x intermediate width
    lin_in = m.DeepLinear(K, F, bias=True, device=DEV, dtype=torch.bfloat16)
    lin_in.fuse_bias = True
    with torch.no_grad():
        lin_in.weight.copy_(bf16(F, K, 1, 0.05))
        lin_in.bias.copy_(bf16(1, F, 2)[0])
    w_down_q, w_down_s = m.weight_quant_block(bf16(K, F // 2, 3, 0.05), dtype=torch.float8_e4m3fn)
    inputs = [bf16(M, K, 10 + i) for i in range(4)]
    with torch.no_grad():
        eager = [mlp_step(x, lin_in, w_down_q, w_down_s).clone() for x in inputs]
        static_x = inputs[0].clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):      # warm-up on the capturing stream: weight cache, library load
            mlp_step(static_x, lin_in, w_down_q, w_down_s)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = mlp_step(static_x, lin_in, w_down_q, w_down_s)
        for i in (1, 2, 3, 0, 2):
            static_x.copy_(inputs[i])
            graph.replay()
            got = static_out.clone()
            torch.cuda.synchronize()
            assert torch.equal(got, eager[i]), (M, i)
            # eager work of the program's own between replays, on the default stream
            again = mlp_step(inputs[(i + 1) % 4], lin_in, w_down_q, w_down_s)
            assert torch.equal(again, eager[(i + 1) % 4]), (M, i)


def test_training_quantizers_and_split_gemm_replay():
    """Backward-path pieces in one graph: both-way quantizers feeding the weight-gradient GEMM (contraction over
    the tokens, a long K against few rows: the K-split path with its fp32 slabs in the workspace)."""
    M, N, K = 8192, 256, 384
    x, dy = bf16(M, K, 21), bf16(M, N, 22)

    def step(x, dy):
        _, _, xq_t, xs_t = m.quant_input(x, only_forward=False)
        _, _, dq_t, ds_t = m.quant_grad_output(dy)
        return m.fp8_matmul(dq_t[:N], ds_t[:N], xq_t[:K], xs_t[:(K + 127) // 128])

    eager = step(x, dy).clone()
    eager2 = step(x * 2, dy).clone()
    sx, sdy = x.clone(), dy.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(sx, sdy)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = step(sx, sdy)
    for rep in range(3):
        sx.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        sx.copy_(x * 2)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager2), rep


def test_calls_from_several_threads_and_streams_do_not_interfere():
    """The library keeps no mutable state between calls: four host threads, each on its own stream, run
    different operators on their own tensors at the same time (ctypes releases the GIL during a call) and
    every result equals the one computed alone."""
    import threading
    torch.manual_seed(5)
    jobs = []
    for i, (M, N, K) in enumerate([(64, 512, 1024), (300, 384, 512), (1, 2048, 2048), (130, 1100, 4224)]):
        x = bf16(M, K, 100 + i)
        w_q, w_s = m.quant_weight(bf16(N, K, 200 + i, 0.05))[:2]

        def job(x=x, w_q=w_q, w_s=w_s, M=M, N=N):
            q, s, _, _ = m.quant_input(x)
            return m.fp8_matmul(q[:M], s[:M], w_q[:N], w_s[:(N + 127) // 128])
        jobs.append(job)
    alone = [j().clone() for j in jobs]
    torch.cuda.synchronize()
    results, errors = [None] * len(jobs), []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(25):
                    out = jobs[i]()
                stream.synchronize()
            results[i] = out
        except Exception as e:        # surfaces in the main thread below
            errors.append(e)
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for got, want in zip(results, alone):
        assert torch.equal(got, want)
