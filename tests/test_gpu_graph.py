"""The ops under HIP graph capture (the reference benchmarks its op inside CUDA graphs,
benchmark/benchmark.py:355-370): moe_align + the fused forward are captured once and replayed
with new inputs; every replay is checked against the eager result of the same inputs, with eager
work and synchronisations between the replays."""
import math

import pytest
import torch

from helpers import reference_routing

pytestmark = pytest.mark.gpu


def _eager(kind, a, ids, wts, E, top_k):
    import prime_moe
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    out = torch.empty((a["x"].shape[0], a["x"].shape[1]), dtype=torch.bfloat16, device=ids.device)
    if kind == "bf16":
        prime_moe.fused_moe_bf16(a["x"], a["w1"], a["w2"], *sched, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
    else:
        prime_moe.fused_moe_mxfp8(a["x"], a["x_scales"], a["w1"], a["w1_scales"], a["w2"], a["w2_scales"],
                                  *sched, wts, out, top_k, 128, 64, 4, 2, 1, True)
    return out


@pytest.mark.parametrize("kind,T,top_k", [
    ("bf16", 192, 2), ("mxfp8", 192, 2),
    ("bf16", 4500, 4),  # 18000 ids: the multi-workgroup moe_align and whole rounds of tiles with a split tail
])
def test_capture_and_replay(kind, T, top_k, device):
    import prime_moe
    K, E, N = 512, 8, 512
    g = torch.Generator(device=device).manual_seed(3)
    w1 = (torch.randn((E, N, K), device=device, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    w2 = (torch.randn((E, K, N // 2), device=device, generator=g) / math.sqrt(N // 2)).to(torch.bfloat16)

    def make_args(x_bf16):
        if kind == "bf16":
            return {"x": x_bf16, "w1": w1, "w2": w2}
        xq, xs = prime_moe.quantize_mx(x_bf16)
        return {"x": xq, "x_scales": xs, "w1": w1q, "w1_scales": w1s, "w2": w2q, "w2_scales": w2s}

    if kind == "mxfp8":
        w1q, s1 = prime_moe.quantize_mx(w1.reshape(E * N, K))
        w2q, s2 = prime_moe.quantize_mx(w2.reshape(E * K, N // 2))
        w1q, w2q = w1q.reshape(E, N, K), w2q.reshape(E, K, N // 2)
        w1s = prime_moe.pack_scales_blocked(s1.reshape(E, N, K // 32))
        w2s = prime_moe.pack_scales_blocked(s2.reshape(E, K, N // 64))

    # static inputs of the graph
    x_static = torch.zeros((T, K), dtype=torch.bfloat16, device=device)
    ids_static = torch.zeros((T, top_k), dtype=torch.int32, device=device)
    wts_static = torch.zeros((T, top_k), dtype=torch.float32, device=device)
    out_static = torch.zeros((T, K), dtype=torch.bfloat16, device=device)

    def body():
        a = make_args(x_static)
        sched = torch.ops.prime_moe.moe_align(ids_static, E, 128, 1)
        if kind == "bf16":
            prime_moe.fused_moe_bf16(a["x"], a["w1"], a["w2"], *sched, wts_static, out_static, top_k,
                                     128, 64, 4, 2, 1, 1, True)
        else:
            prime_moe.fused_moe_mxfp8(a["x"], a["x_scales"], a["w1"], a["w1_scales"], a["w2"], a["w2_scales"],
                                      *sched, wts_static, out_static, top_k, 128, 64, 4, 2, 1, True)

    def new_inputs(seed):
        gg = torch.Generator(device=device).manual_seed(seed)
        x = torch.randn((T, K), device=device, generator=gg).to(torch.bfloat16)
        ids, wts = reference_routing(T, E, top_k, device, gg)
        return x, ids, wts

    x, ids, wts = new_inputs(10)
    x_static.copy_(x); ids_static.copy_(ids); wts_static.copy_(wts)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            body()  # warm-up on the capture stream (allocator pools, library load)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        body()

    for seed in (11, 12, 13, 14):
        x, ids, wts = new_inputs(seed)
        ref = _eager(kind, make_args(x), ids, wts, E, top_k)   # eager work between the replays
        torch.cuda.synchronize()
        x_static.copy_(x); ids_static.copy_(ids); wts_static.copy_(wts)
        out_static.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out_static.float()
        assert torch.isfinite(got).all()
        # same kernels on the same inputs, every sum in a fixed order: the same bits
        assert torch.equal(out_static.view(torch.int16), ref.view(torch.int16)), \
            f"replay with seed {seed} differs from eager"
