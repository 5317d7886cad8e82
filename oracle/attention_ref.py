"""PyTorch (CPU) restatement of the reference's native attention semantics.

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

All functions take CPU tensors and compute in fp32 (or fp64 when
``dtype=torch.float64``) on up-cast inputs: the stated tolerances are against
an fp32 reference.  ``ref_attention(..., reference_dtype_flow=True)`` instead
keeps the reference's dtype flow (matmul in the input dtype, softmax in fp32,
probabilities cast to ``v.dtype`` before P.V, ``areno/accel/attention.py:33-41``),
which differs by one rounding of P for bf16 inputs.
"""

from __future__ import annotations

import torch


def window_left_arg(window_left: int | None) -> int:
    """``None`` means no window; the kernels use -1 (``areno/accel/attention.py:17-18``)."""
    return -1 if window_left is None else int(window_left)


def default_scale(head_dim: int, softmax_scale: float | None) -> float:
    """``areno/accel/attention.py:21-22``."""
    return float(softmax_scale if softmax_scale is not None else head_dim**-0.5)


def ref_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    query_start: int,
    window_left: int,
    softmax_scale: float,
    *,
    dtype: torch.dtype = torch.float32,
    reference_dtype_flow: bool = False,
) -> torch.Tensor:
    """Causal (optionally left-windowed) attention; ``q (.., H, Sq, D)``, ``k, v (.., H, Sk, D)``.

    Follows ``_reference_attention`` (``areno/accel/attention.py:25-41``): query
    ``i`` sits at absolute position ``query_start + i`` and sees key positions
    ``p`` with ``p <= pos`` and, when ``window_left >= 0``, ``p >= pos - window_left``.
    """
    if not reference_dtype_flow:
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    scores = torch.matmul(q, k.transpose(-1, -2)) * softmax_scale
    sq, sk = q.shape[-2], k.shape[-2]
    q_pos = torch.arange(query_start, query_start + sq).view(sq, 1)
    k_pos = torch.arange(sk).view(1, sk)
    mask = k_pos <= q_pos
    if window_left >= 0:
        mask = mask & (k_pos >= q_pos - window_left)
    scores = scores.masked_fill(~mask, torch.finfo(scores.dtype).min)
    if reference_dtype_flow:
        probs = torch.softmax(scores.float(), dim=-1).to(v.dtype)
    else:
        probs = torch.softmax(scores, dim=-1)
    return torch.matmul(probs, v)


def gather_paged(cache: torch.Tensor, block_row: torch.Tensor, length: int) -> torch.Tensor:
    """Rows ``cache[block_row[p // bs], p % bs]`` for ``p in [0, length)`` -> ``(length, Hkv, D...)``.

    The gather of ``_reference_paged_decode_attention`` (``areno/accel/attention.py:57-63``).
    """
    bs = cache.shape[1]
    pos = torch.arange(length)
    ids = block_row.long()[torch.div(pos, bs, rounding_mode="floor")]
    return cache[ids, pos % bs]


def ref_paged_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    cache_seqlens: torch.Tensor,
    window_left: int,
    softmax_scale: float,
    *,
    dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Single-token paged decode; ``q (B, Hq, D)`` -> ``(B, Hq, D)`` in ``dtype``.

    Follows ``_reference_paged_decode_attention`` (``areno/accel/attention.py:44-76``):
    the new token is assumed to be already in the cache, sequence ``b`` has
    ``length = cache_seqlens[b] + 1`` keys, query head ``h`` reads KV head
    ``h // (Hq // Hkv)`` (``repeat_interleave``), the query sits at ``length - 1``.
    Caches must already be floating point (dequantize quantized caches first).
    """
    outs = []
    hq = q.shape[1]
    for b in range(q.shape[0]):
        length = int(cache_seqlens[b]) + 1
        k = gather_paged(k_cache, block_table[b], length)
        v = gather_paged(v_cache, block_table[b], length)
        g = hq // k.shape[1]
        k = k.repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        v = v.repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        out = ref_attention(
            q[b : b + 1].unsqueeze(2), k, v, length - 1, window_left, softmax_scale, dtype=dtype
        )
        outs.append(out.squeeze(2))
    return torch.cat(outs, dim=0)


def ref_decode_update(
    k_update: torch.Tensor,
    v_update: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    cache_seqlens: torch.Tensor,
) -> None:
    """In-place append of one token per sequence.

    ``paged_decode_update_kernel`` (``areno/accel/csrc/attention.cu:526-553``) and
    ``_store_decode_cache`` (``attention_backend/infer.py:266-288``): row ``b`` goes to
    ``cache[block_table[b, L_b // bs], L_b % bs]``.  Rows are applied in order, so when
    several rows alias one slot (graph-padded rows on the scratch block) the last wins.
    """
    bs = k_cache.shape[1]
    for b in range(k_update.shape[0]):
        pos = int(cache_seqlens[b])
        blk = int(block_table[b, pos // bs])
        k_cache[blk, pos % bs] = k_update[b].to(k_cache.dtype)
        v_cache[blk, pos % bs] = v_update[b].to(v_cache.dtype)


def ref_cache_write(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cache_block_ids: torch.Tensor,
    cache_block_offsets: torch.Tensor,
) -> None:
    """``k_cache[ids[t], offs[t]] = key[t]`` for every packed token (same for V).

    ``_store_prefill_cache`` (``attention_backend/infer.py:245-263``); a V narrower than
    the cache head dim is zero-padded first (``common.py:81-90``).
    """
    ids, offs = cache_block_ids.long(), cache_block_offsets.long()
    k_cache.index_put_((ids, offs), key.to(k_cache.dtype))
    if value.shape[-1] != v_cache.shape[-1]:
        padded = value.new_zeros(*value.shape[:-1], v_cache.shape[-1])
        padded[..., : value.shape[-1]] = value
        value = padded
    v_cache.index_put_((ids, offs), value.to(v_cache.dtype))


def ref_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    window_left: int,
    softmax_scale: float,
    *,
    dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Packed causal self-attention over new tokens only; ``q (T,Hq,D)``, ``k,v (T,Hkv,D)``.

    ``varlen_causal_attention_forward_kernel`` (``areno/accel/csrc/attention.cu:145-242``):
    token ``t`` of the sequence starting at ``cu_seqlens[s]`` sees keys
    ``[max(seq_start, t - window_left), t]``; GQA via ``kv_h = h // (Hq // Hkv)``.
    Equivalent to per-sequence ``ref_attention(query_start=0)``.
    """
    out = torch.empty(q.shape, dtype=dtype)
    g = q.shape[1] // k.shape[1]
    cu = [int(x) for x in cu_seqlens]
    for s in range(len(cu) - 1):
        lo, hi = cu[s], cu[s + 1]
        if hi == lo:
            continue
        qs = q[lo:hi].transpose(0, 1).unsqueeze(0)
        ks = k[lo:hi].repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        vs = v[lo:hi].repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        o = ref_attention(qs, ks, vs, 0, window_left, softmax_scale, dtype=dtype)
        out[lo:hi] = o.squeeze(0).transpose(0, 1)
    if cu[-1] < q.shape[0]:
        out[cu[-1] :] = 0
    return out


def ref_paged_varlen_prefill(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    context_lens: torch.Tensor,
    window_left: int,
    softmax_scale: float,
    *,
    dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Causal prefill of ``n_s`` new queries per sequence over ``ctx_s + n_s`` paged keys.

    This build's extension of the path (the reference's chunked prefill never re-reads
    earlier chunks).  The new tokens' KV are already in the cache; query ``i`` of sequence
    ``s`` sits at absolute position ``context_lens[s] + i``.  Per sequence it is
    ``ref_attention(query_start=ctx)`` over the gathered keys, which is exactly how
    ``_reference_attention`` (``areno/accel/attention.py:25-41``) treats a query offset.
    """
    out = torch.zeros(q.shape, dtype=dtype)
    hq = q.shape[1]
    cu = [int(x) for x in cu_seqlens_q]
    for s in range(len(cu) - 1):
        lo, hi = cu[s], cu[s + 1]
        n = hi - lo
        if n == 0:
            continue
        ctx = int(context_lens[s])
        k = gather_paged(k_cache, block_table[s], ctx + n)
        v = gather_paged(v_cache, block_table[s], ctx + n)
        g = hq // k.shape[1]
        k = k.repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        v = v.repeat_interleave(g, dim=1).transpose(0, 1).unsqueeze(0)
        qs = q[lo:hi].transpose(0, 1).unsqueeze(0)
        o = ref_attention(qs, k, v, ctx, window_left, softmax_scale, dtype=dtype)
        out[lo:hi] = o.squeeze(0).transpose(0, 1)
    return out
