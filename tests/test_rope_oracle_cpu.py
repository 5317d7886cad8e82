"""Pins of the RMSNorm / rotary restatement (oracle/rope_ref.py) by what the mathematics fixes."""

import math

import torch

from oracle import rope_ref as rr


def test_rmsnorm_matches_float64_and_is_scale_invariant():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 3, 128, generator=g)
    w = torch.rand(128, generator=g) + 0.5
    got = rr.ref_rmsnorm(x, w, 1e-6)
    x64 = x.double()
    want = x64 / torch.sqrt(x64.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert torch.allclose(got.double(), want, atol=1e-5)
    ones = rr.ref_rmsnorm(x, torch.ones(128), 0.0)
    assert torch.allclose(ones.pow(2).mean(-1), torch.ones(7, 3), atol=1e-5)  # unit RMS
    assert torch.allclose(rr.ref_rmsnorm(3.5 * x, w, 0.0), rr.ref_rmsnorm(x, w, 0.0), atol=1e-5)
    assert rr.ref_rmsnorm(x, None, 1e-6) is x


def test_rope_identity_norm_additivity_and_complex_form():
    d, theta = 64, 10000.0
    cos, sin = rr.rope_tables(d, 512, theta)
    assert cos.shape == (512, d) and torch.equal(cos[:, : d // 2], cos[:, d // 2 :])
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 2, d, generator=g, dtype=torch.float64)
    c64, s64 = cos.double(), sin.double()
    pos = torch.tensor([0, 1, 7, 100, 511])
    y = rr.ref_rope(x, pos, c64, s64)
    assert torch.equal(y[0], x[0])  # position 0: cos = 1, sin = 0
    # every (i, i + D/2) pair is rotated: its length is preserved
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2 :] ** 2  # noqa: E731
    assert torch.allclose(pair(y), pair(x), atol=1e-5)
    # rotations add: rope(p1) then rope(p2) == rope(p1 + p2)
    p1, p2 = torch.tensor([3, 10, 20, 30, 40]), torch.tensor([5, 1, 100, 200, 300])
    twice = rr.ref_rope(rr.ref_rope(x, p1, c64, s64), p2, c64, s64)
    assert torch.allclose(twice, rr.ref_rope(x, p1 + p2, c64, s64), atol=2e-4)  # tables are float32, angles up to 340 rad
    # complex form: (x1 + i x2) * exp(i p w_j) with w_j = theta^(-2j/D)
    w = torch.tensor([theta ** (-2.0 * j / d) for j in range(d // 2)], dtype=torch.float64)
    z = torch.complex(x[..., : d // 2], x[..., d // 2 :]) * torch.exp(1j * pos.double()[:, None, None] * w)
    assert torch.allclose(y[..., : d // 2], z.real, atol=2e-4) and torch.allclose(y[..., d // 2 :], z.imag, atol=2e-4)
    assert math.isclose(float(cos[1, 0]), math.cos(1.0), rel_tol=1e-6)


def test_rope_rounds_like_the_eager_ops_in_bf16():
    d = 128
    cos, sin = rr.rope_tables(d, 64, 10000.0)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 3, d, generator=g).bfloat16()
    pos = torch.tensor([1, 2, 33, 63])
    got = rr.ref_rope(x, pos, cos, sin)
    assert got.dtype == torch.bfloat16
    # explicit rounding of each product and of the sum
    c, s = cos[pos].unsqueeze(1).bfloat16().float(), sin[pos].unsqueeze(1).bfloat16().float()
    xf = x.float()
    a = (xf * c).bfloat16().float()
    b = (rr.rotate_half(xf) * s).bfloat16().float()
    assert torch.equal(got, (a + b).bfloat16())
