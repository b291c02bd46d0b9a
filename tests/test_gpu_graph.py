"""The ops under HIP graph capture (the reference benchmarks its op inside CUDA graphs,
benchmark/benchmark.py:355-370) and under torch's tracing (the reference registers fake impls for
that, prime_moe/__init__.py:5-24, :51-72): moe_align + the fused forward are captured once and
replayed with new inputs; every replay is checked against the CPU oracle and, bit for bit, against
the eager result of the same inputs, with eager work and synchronisations between the replays."""
import math

import pytest
import torch

from helpers import BF16_GATE, MX_COS_GATE, MX_RELL2_GATE, cosine, reference_routing, rel_clamp, rel_l2
from oracle import moe_oracle as O

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
    ("mxfp8", 4500, 4),
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
        # and the replay against the CPU oracle on the same inputs
        if kind == "bf16":
            want = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())
            assert rel_clamp(got.cpu(), want, 1.0) <= BF16_GATE, f"replay with seed {seed} vs oracle"
        else:
            a = make_args(x)
            deq = lambda q, sc: O.dequantize_mx_torch(q.cpu(), sc.view(torch.uint8).cpu())
            want = O.fused_moe_dense(deq(a["x"], a["x_scales"]), deq(w1q, s1.reshape(E, N, K // 32)),
                                     deq(w2q, s2.reshape(E, K, N // 64)), ids.cpu(), wts.cpu(), act_mx=True)
            assert cosine(got.cpu(), want) >= MX_COS_GATE and rel_l2(got.cpu(), want) <= MX_RELL2_GATE, \
                f"replay with seed {seed} vs oracle"


def _small_case(kind, device, T=96, K=512, E=4, N=512, top_k=2, seed=21):
    import prime_moe
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn((T, K), device=device, generator=g).to(torch.bfloat16)
    w1 = (torch.randn((E, N, K), device=device, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    w2 = (torch.randn((E, K, N // 2), device=device, generator=g) / math.sqrt(N // 2)).to(torch.bfloat16)
    ids, wts = reference_routing(T, E, top_k, device, g)
    if kind == "bf16":
        return dict(x=x, w1=w1, w2=w2, ids=ids, wts=wts, E=E, top_k=top_k)
    xq, xs = prime_moe.quantize_mx(x)
    w1q, s1 = prime_moe.quantize_mx(w1)
    w2q, s2 = prime_moe.quantize_mx(w2)
    return dict(x=xq, x_scales=xs, w1=w1q, w1_scales=prime_moe.pack_scales_blocked(s1), w2=w2q,
                w2_scales=prime_moe.pack_scales_blocked(s2), ids=ids, wts=wts, E=E, top_k=top_k)


def test_opcheck_all_three_ops(device):
    """torch.library.opcheck: schema (the declared mutation of `out` and nothing else), fake impls that
    agree with the real outputs in shape / dtype / device, and AOT dispatch with dynamic shapes."""
    import prime_moe  # noqa: F401
    c = _small_case("bf16", device)
    torch.library.opcheck(torch.ops.prime_moe.moe_align.default, (c["ids"], c["E"], 128, 1))
    sched = torch.ops.prime_moe.moe_align(c["ids"], c["E"], 128, 1)
    for split in (True, False):
        out = torch.zeros_like(c["x"])
        torch.library.opcheck(torch.ops.prime_moe.fused_moe_bf16.default,
                              (c["x"], c["w1"], c["w2"], *sched, c["wts"], out, c["top_k"], 128, 64, 4, 2, 1, 1, split))
    m = _small_case("mxfp8", device)
    sched = torch.ops.prime_moe.moe_align(m["ids"], m["E"], 128, 1)
    out = torch.zeros((m["x"].shape[0], m["x"].shape[1]), dtype=torch.bfloat16, device=device)
    # (without opcheck's schema test here: it perturbs its inputs with a multiplication, which torch
    # does not implement for float8_e4m3fn tensors; the schema string itself is asserted in test_host.py)
    torch.library.opcheck(torch.ops.prime_moe.fused_moe_mxfp8.default,
                          (m["x"], m["x_scales"], m["w1"], m["w1_scales"], m["w2"], m["w2_scales"], *sched, m["wts"],
                           out, m["top_k"], 128, 64, 4, 2, 1, True),
                          test_utils=("test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic"))


@pytest.mark.parametrize("kind", ["bf16", "mxfp8"])
def test_torch_compile_matches_eager(kind, device):
    """The three ops traced by torch.compile (aot_eager backend, fullgraph: no graph break at any of
    them, which needs the fake impls) give the bits of the eager calls."""
    import prime_moe
    c = _small_case(kind, device, T=300, top_k=3, seed=22)
    E, top_k = c["E"], c["top_k"]

    def forward(ids, wts, x):
        s, e, n = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
        out = torch.zeros((x.shape[0], x.shape[1]), dtype=torch.bfloat16, device=x.device)
        if kind == "bf16":
            torch.ops.prime_moe.fused_moe_bf16(x, c["w1"], c["w2"], s, e, n, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
            torch.ops.prime_moe.fused_moe_bf16(x, c["w1"], c["w2"], s, e, n, wts, out, top_k, 128, 64, 4, 2, 1, 1, False)
        else:
            torch.ops.prime_moe.fused_moe_mxfp8(x, c["x_scales"], c["w1"], c["w1_scales"], c["w2"], c["w2_scales"],
                                                s, e, n, wts, out, top_k, 128, 64, 4, 2, 1, True)
            torch.ops.prime_moe.fused_moe_mxfp8(x, c["x_scales"], c["w1"], c["w1_scales"], c["w2"], c["w2_scales"],
                                                s, e, n, wts, out, top_k, 128, 64, 4, 2, 1, False)
        return out.float() * 0.5  # split=True result, plus the same again accumulated by split=False, halved

    eager = forward(c["ids"], c["wts"], c["x"])
    compiled = torch.compile(forward, backend="aot_eager", fullgraph=True)
    got = compiled(c["ids"], c["wts"], c["x"])
    torch.cuda.synchronize()
    assert torch.isfinite(got).all() and float(got.abs().max()) > 0
    assert torch.equal(got, eager)
    # a second call of the compiled function with other routing: no stale state in the traced graph
    ids2, wts2 = reference_routing(300, E, top_k, device, torch.Generator(device=device).manual_seed(23))
    assert torch.equal(compiled(ids2, wts2, c["x"]), forward(ids2, wts2, c["x"]))
