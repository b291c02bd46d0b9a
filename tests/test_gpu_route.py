"""prime_moe.route (top-k + softmax + moe_align on the GPU, through the C ABI) vs the CPU oracle:
expert ids and the three moe_align outputs bit-exact, weights within 1e-6."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

W_TOL = 1e-6  # absolute, on softmax weights in [0, 1]


def _check(logits: torch.Tensor, top_k: int, bias=None, block_m=128, bpc=1):
    import prime_moe
    ids, w, s, e, t = prime_moe.route(logits, top_k, block_m, bpc, bias=bias)
    torch.cuda.synchronize()
    E = logits.shape[1]
    ref_ids, ref_w = O.route_topk(logits.float().cpu().numpy(), top_k,
                                  bias.cpu().numpy() if bias is not None else None)
    np.testing.assert_array_equal(ids.cpu().numpy(), ref_ids, err_msg="topk_ids")
    assert float(np.abs(w.cpu().numpy().astype(np.float64) - ref_w).max(initial=0.0)) <= W_TOL
    for got, want, name in zip((s, e, t), O.moe_align_fast(ref_ids, E, block_m, bpc),
                               ("sorted_token_ids", "expert_ids", "num_tokens_post_padded")):
        np.testing.assert_array_equal(got.cpu().numpy(), want, err_msg=name)
    return ids, w, s, e, t


@pytest.mark.parametrize("name", ["c1_readme_bf16", "c2_mixtral_bf16", "c3_qwen3_bf16", "c4_dsv3_mxfp8"])
def test_route_on_benchmark_routings(name, device):
    # the gate logits of the benchmark configurations (those that route by top-k of logits)
    from prime_moe.workloads import CONFIGS
    cfg = CONFIGS[name]
    g = torch.Generator(device=device).manual_seed(1)
    if cfg.routing == "uniform":
        logits = torch.rand((cfg.T, cfg.E), generator=g, device=device)
    else:
        logits = torch.randn((cfg.T, cfg.E), generator=g, device=device)
    bias = 0.5 * torch.randn((cfg.E,), generator=g, device=device) if cfg.routing == "topk_bias" else None
    ids, w, *_ = _check(logits, cfg.top_k, bias=bias)
    # and against torch's own top-k + softmax (what the unfused sequence computes)
    v = logits if bias is None else logits + bias
    vals, idx = torch.topk(v, cfg.top_k, dim=-1)
    same_rows = (idx.to(torch.int32) == ids).all(dim=1)  # rows with ties may legitimately differ in order
    assert float(same_rows.float().mean()) > 0.999
    torch.testing.assert_close(w[same_rows], torch.softmax(vals.float(), -1)[same_rows], rtol=0, atol=2e-6)


def test_route_decode_shape_and_zipf_popularity(device):
    # C5-like: 64 tokens, 256 experts, logits = log popularity + Gumbel noise (top-k of these samples
    # experts without replacement in proportion to popularity)
    g = torch.Generator(device=device).manual_seed(2)
    pop = torch.arange(1, 257, device=device, dtype=torch.float32).pow(-1.2)
    u = torch.rand((64, 256), generator=g, device=device).clamp_min(1e-9)
    _check(pop.log() - (-u.log()).log(), 8)


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (3, 2, 2), (65, 64, 1), (17, 65, 9), (9, 257, 9), (4, 1024, 32),
                                   (1000, 37, 9), (40000, 8, 2)])
def test_route_shapes(T, E, k, device):
    g = torch.Generator(device=device).manual_seed(T + E + k)
    _check(torch.randn((T, E), generator=g, device=device), k)


def test_route_ties_go_to_the_lower_index(device):
    # few distinct values: almost every selection is decided by the tie rule
    g = torch.Generator(device=device).manual_seed(3)
    logits = torch.randint(-2, 3, (512, 200), generator=g, device=device).float()
    logits[0] = 0.0
    logits[1, ::2] = -0.0  # -0 ties with +0
    _check(logits, 8)
    _check(torch.zeros((5, 1024), device=device), 32)


def test_route_bf16_logits_bias_and_special_values(device):
    g = torch.Generator(device=device).manual_seed(4)
    logits = torch.randn((300, 128), generator=g, device=device)
    _check(logits.to(torch.bfloat16), 8)
    _check(logits.to(torch.bfloat16), 8, bias=torch.randn((128,), generator=g, device=device))
    # infinities order like numbers; rows stay finite in the softmax as long as the maximum is finite
    logits[0, 5] = float("-inf")
    logits[1, :120] = float("-inf")
    _check(logits, 8)
    # other block sizes of the align step
    _check(logits, 4, block_m=16, bpc=2)


def test_route_nan_ranks_above_numbers(device):
    import prime_moe
    logits = torch.tensor([[0.0, float("nan"), 3.0, float("inf")]], device=device)
    ids, _, *_ = prime_moe.route(logits, 3)
    assert ids.cpu().tolist() == [[1, 3, 2]]


def test_route_feeds_the_fused_op(device):
    # end to end: route -> fused_moe_bf16 equals topk/softmax/moe_align -> fused_moe_bf16 bit for bit
    import prime_moe
    g = torch.Generator(device=device).manual_seed(5)
    T, K, E, N, k = 200, 512, 16, 512, 4
    x = torch.randn((T, K), generator=g, device=device).to(torch.bfloat16)
    w1 = (torch.randn((E, N, K), generator=g, device=device) / K ** 0.5).to(torch.bfloat16)
    w2 = (torch.randn((E, K, N // 2), generator=g, device=device) / (N // 2) ** 0.5).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g, device=device)
    ids, w, s, e, t = prime_moe.route(logits, k)
    out_a = torch.empty((T, K), dtype=torch.bfloat16, device=device)
    prime_moe.fused_moe_bf16(x, w1, w2, s, e, t, w, out_a, k, 128, 64, 4, 2)
    ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), w.cpu())
    err = float(((out_a.float().cpu() - ref).abs() / ref.abs().clamp_min(1.0)).max())
    assert err <= 2e-2


def test_route_errors(device):
    import prime_moe
    logits = torch.zeros((4, 8), device=device)
    for bad in (dict(top_k=0), dict(top_k=9), dict(top_k=2, block_m=0)):
        with pytest.raises(RuntimeError):
            prime_moe.route(logits, **bad)
    with pytest.raises(RuntimeError):
        prime_moe.route(logits.double(), 2)
    with pytest.raises(RuntimeError):
        prime_moe.route(logits.cpu(), 2)
    with pytest.raises(RuntimeError):
        prime_moe.route(logits.t(), 2)
    with pytest.raises(RuntimeError):
        prime_moe.route(logits, 2, bias=torch.zeros((8,)))
    with pytest.raises(RuntimeError):
        prime_moe.route(torch.zeros((2, 1025), device=device), 2)
