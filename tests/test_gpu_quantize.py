"""GPU OCP-MX quantiser (the routine shared with the on-chip activation requantisation) vs
the bit-level CPU oracle: codes and scales bit-exact."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _check(x_bf16: torch.Tensor):
    import prime_moe
    q, s = prime_moe.quantize_mx(x_bf16)
    torch.cuda.synchronize()
    qr, sr = O.quantize_mx(x_bf16.float().cpu().numpy())
    np.testing.assert_array_equal(s.view(torch.uint8).cpu().numpy(), sr)
    got = q.view(torch.uint8).cpu().numpy()
    # +0 / -0 are distinct codes with equal value; the hardware keeps the sign of a zero product
    np.testing.assert_array_equal(O.e4m3_decode(got), O.e4m3_decode(qr))
    nz = O.e4m3_decode(qr) != 0
    np.testing.assert_array_equal(got[nz], qr[nz])


def test_quantize_random(device):
    g = torch.Generator(device=device).manual_seed(0)
    x = torch.randn((257, 4096), device=device, generator=g)
    x = x * torch.tensor([1e-3, 1.0, 37.0, 1e4], device=device).repeat(1024)[None, :]
    _check(x.to(torch.bfloat16))


def test_quantize_known_answers_and_ties(device):
    vals = [0.0, 1.0, 3.5, 3.90625, 448.0, 449.0, 510.0, 512.0, -3.5, 2.0 ** -120, 1.0625, 1.1875, 17.0, 19.0]
    rows = []
    for v in vals:
        b = torch.zeros(32)
        b[0] = v
        rows.append(b)
    # tie cases inside a block whose maximum fixes the scale at 2^-8 * ... : max 256 -> e = 127
    b = torch.tensor([256.0, 17.0, 19.0, 1.0625 * 16, 1.1875 * 16, 2.0 ** -10, 3 * 2.0 ** -10] + [0.0] * 25)
    rows.append(b)
    _check(torch.stack(rows).to(torch.bfloat16).to(device))


def test_quantize_shapes(device):
    import prime_moe
    x = torch.randn((3, 5, 64), device=device).to(torch.bfloat16)
    q, s = prime_moe.quantize_mx(x)
    assert q.shape == (3, 5, 64) and q.dtype == torch.float8_e4m3fn
    assert s.shape == (3, 5, 2) and s.dtype == torch.float8_e8m0fnu
    with pytest.raises(RuntimeError):
        prime_moe.quantize_mx(x[..., :48].contiguous())
    with pytest.raises(RuntimeError):
        prime_moe.quantize_mx(x.float())
