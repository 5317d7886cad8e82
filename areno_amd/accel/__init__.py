"""Paged / quantized KV-cache attention ops (the hot path of ``areno.accel`` in the reference).

Re-exports the op surface the reference's inference backend imports
(``areno/accel/__init__.py:17-21`` there) plus this build's additions (cache write, paged prefill, the fused
QK-norm + rotary + cache-write step in front of the path, and what a decode step prepares once for all its layers:
the plan of the decode op and the rotary rows of the fused step).
"""

from areno_amd.accel.attention import (
    areno_causal_attention,
    areno_paged_cache_write,
    areno_paged_causal_attention_decode,
    areno_paged_decode_plan,
    areno_paged_varlen_causal_attention,
    areno_qk_norm_rope_cache_write,
    areno_rope_rows,
    areno_varlen_causal_attention,
)

__all__ = [
    "areno_causal_attention",
    "areno_paged_cache_write",
    "areno_paged_causal_attention_decode",
    "areno_paged_decode_plan",
    "areno_paged_varlen_causal_attention",
    "areno_qk_norm_rope_cache_write",
    "areno_rope_rows",
    "areno_varlen_causal_attention",
]
