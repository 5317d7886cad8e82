"""Paged KV-cache pools, one pair per layer, shaped ``[blocks, block_size, local_kv_heads, head_dim]`` like the
reference's ``allocate_kv_caches`` (areno/models/qwen3/model.py:309-333), plus the per-token-per-head scale pools
``[blocks, block_size, local_kv_heads]`` an int8 / fp8 cache needs."""

from __future__ import annotations

from dataclasses import dataclass

import torch

_QUANTIZED = {
    "int8": (torch.int8, torch.float16),
    "fp8": (torch.float8_e4m3fn, torch.float32),
}


@dataclass(slots=True)
class KVCacheLayer:
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    k_scale: torch.Tensor | None = None
    v_scale: torch.Tensor | None = None

    @property
    def quantized(self) -> bool:
        return self.k_scale is not None

    def as_tuple(self) -> tuple[torch.Tensor, torch.Tensor]:
        """The ``(k_cache, v_cache)`` pair the reference's layers keep."""
        return self.k_cache, self.v_cache


def _resolve(dtype: torch.dtype, kv_cache_dtype: str) -> tuple[torch.dtype, torch.dtype | None]:
    if kv_cache_dtype in ("auto", "model"):
        return dtype, None
    if kv_cache_dtype in _QUANTIZED:
        return _QUANTIZED[kv_cache_dtype]
    raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}; expected 'auto', 'int8' or 'fp8'")


def allocate_kv_caches(
    num_layers: int,
    num_blocks: int,
    block_size: int,
    local_kv_heads: int,
    head_dim: int,
    device: torch.device | str,
    dtype: torch.dtype,
    kv_cache_dtype: str = "auto",
) -> list[KVCacheLayer]:
    """``num_blocks`` counts the scratch block the decode graph parks padded rows on, as in the reference
    (areno/engine/runtime/decode_graph.py:89-96 allocates ``num_blocks + 1`` and uses the last)."""
    if min(num_layers, num_blocks, block_size, local_kv_heads, head_dim) <= 0:
        raise ValueError("cache geometry must be positive")
    cache_dtype, scale_dtype = _resolve(dtype, kv_cache_dtype)
    layers = []
    for _ in range(num_layers):
        shape = (num_blocks, block_size, local_kv_heads, head_dim)
        k_cache = torch.empty(shape, device=device, dtype=cache_dtype)
        v_cache = torch.empty(shape, device=device, dtype=cache_dtype)
        k_scale = v_scale = None
        if scale_dtype is not None:
            # scale 1 with code 0 reads as 0.0: a never-written slot that a padded row touches stays finite
            k_cache.view(torch.uint8).zero_()
            v_cache.view(torch.uint8).zero_()
            k_scale = torch.ones(shape[:3], device=device, dtype=scale_dtype)
            v_scale = torch.ones(shape[:3], device=device, dtype=scale_dtype)
        layers.append(KVCacheLayer(k_cache, v_cache, k_scale, v_scale))
    return layers


def kv_cache_bytes_per_token(local_kv_heads: int, head_dim: int, dtype: torch.dtype, kv_cache_dtype: str = "auto") -> int:
    """Bytes one cached token costs in one layer (K and V, codes and scales): what the block manager divides the
    HBM budget by."""
    cache_dtype, scale_dtype = _resolve(dtype, kv_cache_dtype)
    per_head = head_dim * torch.empty((), dtype=cache_dtype).element_size()
    if scale_dtype is not None:
        per_head += torch.empty((), dtype=scale_dtype).element_size()
    return 2 * local_kv_heads * per_head
