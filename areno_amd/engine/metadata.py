"""Attention metadata for one inference forward call.

Same fields and meaning as the reference's ``InferMeta`` (areno/engine/runtime/metadata.py:29-45); ``context_lens`` is
the one addition: tokens of each sequence that were cached by earlier prefill chunks, which lets a later chunk attend
to them (the reference's chunked prefill only sees the chunk itself, areno/engine/data/rollout_state.py:121-172).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

import torch


@dataclass(slots=True)
class InferMeta:
    """Prefill: ``cu_seqlens`` / ``max_seqlen`` over the packed new tokens, ``cache_block_ids`` /
    ``cache_block_offsets`` = where each new token's K/V goes, ``block_table`` (and ``context_lens`` for chunks that
    continue a cached sequence).  Decode: one row per active sequence, ``cache_seqlens`` = tokens already cached,
    ``block_table`` = logical block -> pool block."""

    mode: Literal["prefill", "decode"]
    sample_indices: torch.Tensor | None = None
    cu_seqlens: torch.Tensor | None = None
    max_seqlen: int | None = None
    cache_seqlens: torch.Tensor | None = None
    block_table: torch.Tensor | None = None
    cache_block_ids: torch.Tensor | None = None
    cache_block_offsets: torch.Tensor | None = None
    context_lens: torch.Tensor | None = None
