"""The backward oracle is torch autograd through the oracle's forward; this pins that the forward is differentiable
as written (in-place assembly of the packed output included) and that autograd's gradients equal finite differences."""

import torch

from oracle import attention_ref as ar


def test_autograd_of_the_varlen_oracle_equals_finite_differences():
    g = torch.Generator().manual_seed(1)
    cu = torch.tensor([0, 3, 3, 8], dtype=torch.int32)
    q = torch.randn(8, 4, 6, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(8, 2, 6, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(8, 2, 6, generator=g, dtype=torch.float64, requires_grad=True)
    for window in (-1, 2):
        fn = lambda a, b, c: ar.ref_varlen(a, b, c, cu, window, 0.4, dtype=torch.float64)  # noqa: E731
        assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-6)


def test_autograd_of_the_dense_oracle_equals_finite_differences():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 2, 3, 4, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(2, 2, 7, 4, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(2, 2, 7, 4, generator=g, dtype=torch.float64, requires_grad=True)
    fn = lambda a, b, c: ar.ref_attention(a, b, c, 2, 3, 0.5, dtype=torch.float64)  # noqa: E731
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-6)
