"""CPU restatement of the layer steps in front of the attention path.  TEST INFRASTRUCTURE ONLY.

* ``ref_rmsnorm``: ``rmsnorm_forward_kernel`` (``areno/accel/csrc/normalization.cu:34-56``):
  ``y = dtype(float(x) * rsqrt(mean(float(x)^2) + eps) * w)`` with an fp32 weight.
* ``rope_tables`` / ``ref_rope``: ``RotaryEmbedding`` (``areno/engine/layers/rotary.py:17-52``): fp32 tables
  ``cos/sin(outer(pos, theta^(-2i/D)))`` doubled to the full head dim, cast to the activation dtype at use;
  ``out = x * cos + rotate_half(x) * sin`` evaluated with the activation dtype's eager tensor ops, i.e. each product
  and the sum rounded to that dtype.
"""

from __future__ import annotations

import torch


def ref_rmsnorm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    """Per-row RMSNorm over the last dim in fp32, result in ``x.dtype``; ``weight=None`` returns ``x`` (no norm)."""
    if weight is None:
        return x
    xf = x.float()
    inv = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xf * inv * weight.float()).to(x.dtype)


def rope_tables(head_dim: int, max_position: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """``cos_cached`` / ``sin_cached`` of shape ``(max_position, head_dim)``, float32 (rotary.py:34-44)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(max_position, dtype=torch.float32), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def ref_rope(x: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``x (T, H, D)`` in its own dtype, ``positions (T,)``; the arithmetic runs in ``x.dtype`` like the eager ops."""
    c = cos[positions].unsqueeze(1).to(x.dtype)
    s = sin[positions].unsqueeze(1).to(x.dtype)
    return (x * c) + (rotate_half(x) * s)


def ref_qk_norm_rope(q, k, positions, cos, sin, q_weight, k_weight, eps):
    """``(q', k')`` as the attention layer computes them (areno/engine/layers/attention.py:90-96)."""
    return (ref_rope(ref_rmsnorm(q, q_weight, eps), positions, cos, sin),
            ref_rope(ref_rmsnorm(k, k_weight, eps), positions, cos, sin))  # fmt: skip
