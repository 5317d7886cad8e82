"""Inference attention backend over the paged, optionally quantized KV cache.

Same call shape as the reference's ``FlashAttnInferBackend.forward``
(areno/engine/layers/attention_backend/infer.py:50-153): ``q (1, T, Hq, D)``, ``k`` / ``v (1, T, Hkv, D)``, the layer's
cache pools and an ``InferMeta``; two extra keyword arguments carry the scale pools of an int8 / fp8 cache.

- prefill: the new K/V rows are quantized and scattered into the pages by ``(block_id, offset)``
  (``areno_paged_cache_write`` in place of the ``index_put_`` pair of infer.py:245-263), then causal attention runs
  over the packed new tokens (``areno_varlen_causal_attention``, infer.py:189-209) or, when the metadata carries
  ``context_lens``, over the pages so a later chunk sees the earlier ones.
- decode: one token per sequence; the op appends it to the page and attends over the whole history
  (``areno_paged_causal_attention_decode``, infer.py:212-242).
"""

from __future__ import annotations

import torch
from torch import nn

from areno_amd.accel.attention import (
    areno_paged_cache_write,
    areno_paged_causal_attention_decode,
    areno_paged_varlen_causal_attention,
    areno_varlen_causal_attention,
)
from areno_amd.engine.metadata import InferMeta


def pad_last_dim(x: torch.Tensor, size: int) -> torch.Tensor:
    """Zero-pad the value head dim to the cache head dim (areno/engine/layers/attention_backend/common.py:81-90)."""
    if x.shape[-1] > size:
        raise ValueError(f"cannot fit last dim {x.shape[-1]} into target dim {size}")
    if x.shape[-1] == size:
        return x
    out = x.new_zeros(*x.shape[:-1], size)
    out[..., : x.shape[-1]] = x
    return out


def _window_left(window_size: tuple[int, int] | None) -> int | None:
    """(-1, -1) or None = full attention; otherwise (left, 0) (infer.py:180-185)."""
    if window_size is None or tuple(window_size) == (-1, -1):
        return None
    if window_size[1] != 0:
        raise ValueError("native attention backend only supports causal right window 0")
    return int(window_size[0])


class HipInferBackend(nn.Module):
    """Prefill and single-token decode on the HIP kernels; stateless apart from the module identity."""

    def forward(
        self,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        k_cache: torch.Tensor,
        v_cache: torch.Tensor,
        meta: InferMeta,
        window_size: tuple[int, int] | None = None,
        softmax_scale: float | None = None,
        update_cache: bool = True,
        k_scale: torch.Tensor | None = None,
        v_scale: torch.Tensor | None = None,
    ) -> torch.Tensor:
        q_flat = q.reshape(-1, q.shape[-2], q.shape[-1])
        k_flat = k.reshape(-1, k.shape[-2], k.shape[-1])
        v_flat = v.reshape(-1, v.shape[-2], v.shape[-1])
        value_dim = int(v_flat.shape[-1])
        qk_dim = int(q_flat.shape[-1])
        window_left = _window_left(window_size)
        if (k_scale is None) != (v_scale is None):
            raise ValueError("k_scale and v_scale must be given together")

        if meta.mode == "prefill":
            if meta.cu_seqlens is None or meta.max_seqlen is None or meta.block_table is None:
                raise ValueError("prefill inference requires cu_seqlens, max_seqlen, block_table")
            v_pad = pad_last_dim(v_flat, qk_dim)
            if update_cache:
                if meta.cache_block_ids is None or meta.cache_block_offsets is None:
                    raise ValueError("prefill inference requires cache_block_ids and cache_block_offsets")
                areno_paged_cache_write(
                    k_flat.contiguous(), pad_last_dim(v_flat, v_cache.shape[-1]).contiguous(), k_cache, v_cache,
                    meta.cache_block_ids, meta.cache_block_offsets, k_scale=k_scale, v_scale=v_scale,
                )  # fmt: skip
            if meta.context_lens is not None:
                # reads the new tokens from the pages: with update_cache=False the caller has already stored them
                # (the fused norm + rotary + cache-write op does)
                out = areno_paged_varlen_causal_attention(
                    q_flat.contiguous(), k_cache, v_cache, meta.block_table.contiguous(), meta.cu_seqlens.contiguous(),
                    meta.context_lens.contiguous(), window_left=window_left, softmax_scale=softmax_scale,
                    k_scale=k_scale, v_scale=v_scale,
                )  # fmt: skip
            else:
                out = areno_varlen_causal_attention(
                    q_flat.contiguous(), k_flat.contiguous(), v_pad.contiguous(), meta.cu_seqlens.contiguous(),
                    window_left=window_left, softmax_scale=softmax_scale,
                )  # fmt: skip
            out = out[..., :value_dim] if out.shape[-1] != value_dim else out
            return out.reshape(q.shape[0], q.shape[1], q.shape[2], value_dim)

        if meta.mode == "decode":
            if meta.cache_seqlens is None or meta.block_table is None:
                raise ValueError("decode inference requires cache_seqlens and block_table")
            if not update_cache:
                raise ValueError("native decode requires update_cache=True")
            if meta.cache_seqlens.dtype != torch.int32:
                raise ValueError("native decode requires int32 cache_seqlens")
            if meta.block_table.dtype != torch.int32:
                raise ValueError("native decode requires int32 block_table")
            out = areno_paged_causal_attention_decode(
                q_flat.contiguous(), k_flat.contiguous(), pad_last_dim(v_flat, v_cache.shape[-1]).contiguous(),
                k_cache, v_cache, meta.block_table.contiguous(), meta.cache_seqlens.contiguous(),
                window_left=window_left, num_splits=8, softmax_scale=softmax_scale,
                k_scale=k_scale, v_scale=v_scale,
            ).to(dtype=q.dtype)  # fmt: skip
            out = out[..., :value_dim] if out.shape[-1] != value_dim else out
            return out.reshape(q.shape[0], q.shape[1], q.shape[2], value_dim)

        raise ValueError(f"unsupported inference mode: {meta.mode}")


def build_infer_attention_backend(attn_backend: str = "native") -> HipInferBackend:
    """Counterpart of the reference's factory (infer.py:156-159); ``"native"`` and ``"flash"`` both resolve to the
    HIP kernels here, there is no other backend."""
    if attn_backend not in ("native", "flash"):
        raise ValueError(f"unsupported attn_backend {attn_backend!r}")
    return HipInferBackend()
