"""Python op surface of the paged / quantized KV-cache attention path.

Drop-in for the ops the reference engine imports from ``areno.accel.attention``
(``areno/engine/layers/attention_backend/infer.py:25`` there):

* ``areno_paged_causal_attention_decode``  (reference ``areno/accel/attention.py:267-314``)
* ``areno_varlen_causal_attention``        (reference ``areno/accel/attention.py:186-209``)
* ``areno_causal_attention``               (reference ``areno/accel/attention.py:121-142``; no engine caller)

with the same positional/keyword arguments, defaults (``window_left=None`` -> no window,
``softmax_scale=None`` -> ``head_dim ** -0.5``, l.17-22 there) and error behaviour
(non-GPU tensor -> ``RuntimeError``; wrong rank or non-int32 metadata -> ``ValueError``;
everything else -> ``RuntimeError`` from the extension's checks).  Keyword-only additions, all
defaulting to the reference behaviour:

* ``k_scale`` / ``v_scale`` on the decode op: per-(token, kv head) scale pools ``[NB, bs, Hkv]``
  for ``int8`` / ``float8_e4m3fn`` caches; the fused cache append then quantizes ``k_update``/``v_update``.
* ``areno_paged_cache_write``: the prefill cache store (``_store_prefill_cache``,
  ``attention_backend/infer.py:245-263`` there) as one quantize-and-scatter kernel.
* ``areno_paged_varlen_causal_attention``: causal prefill of new queries over paged KV with a cached
  context (chunked prefill that re-reads earlier chunks).

Everything runs as HIP kernels through ``areno_amd.accel._areno_accel``; there is no Python
fallback.  The varlen and dense ops are autograd functions with HIP backward kernels like the
reference's; the decode op's backward recomputes densely, as the reference's does; the paged prefill op (this
build's own) is inference-only and refuses inputs that require gradients while gradients are being recorded,
instead of returning an output without a graph.  float64 tensors are accepted as in the reference, whose kernels
read doubles and compute in fp32: the ops run on fp32 copies and cast the result back.
"""

from __future__ import annotations

import torch

from areno_amd.accel._extension import extension as _extension

_QUANTIZED = (torch.int8, torch.float8_e4m3fn)


def _window_left(window_left: int | None) -> int:
    return -1 if window_left is None else int(window_left)


def _scale(q: torch.Tensor, softmax_scale: float | None) -> float:
    return float(softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5)


def _all_on_gpu(*tensors: torch.Tensor | None) -> bool:
    return all(t.is_cuda for t in tensors if t is not None)


def _contig(t: torch.Tensor | None) -> torch.Tensor | None:
    return None if t is None else t.contiguous()


def _no_autograd(op: str, *tensors: torch.Tensor | None) -> None:
    """The paged prefill op (this build's own; the reference has none) has no backward.  Rather than hand back an
    output that silently carries no gradient, a call that autograd would have to record is refused."""
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise RuntimeError(
            f"{op}: backward is not implemented for the paged prefill op; call it under torch.no_grad() / "
            "torch.inference_mode() or detach the inputs"
        )


def _check_scales(op: str, cache: torch.Tensor, k_scale, v_scale) -> None:
    if (k_scale is None) != (v_scale is None):
        raise ValueError(f"{op} expects k_scale and v_scale together")
    if cache.dtype in _QUANTIZED and k_scale is None:
        raise ValueError(f"{op} expects k_scale and v_scale for an int8/float8_e4m3fn cache")
    if cache.dtype not in _QUANTIZED and k_scale is not None:
        raise ValueError(f"{op} got scales for an unquantized cache")
    if k_scale is not None and (k_scale.dim() != 3 or v_scale.dim() != 3):
        raise ValueError(f"{op} expects scales shaped (num_blocks, block_size, kv_heads)")


class _VarlenCausalAttention(torch.autograd.Function):
    """Forward and backward of the packed varlen op, as ``_ArenoVarlenCausalAttention`` in the reference
    (``areno/accel/attention.py:145-183``): the forward saves q, k, v, the output and cu_seqlens; the backward kernels
    return fp32 gradients that are cast to the inputs' dtypes."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, window_left: int, softmax_scale: float):
        out = _extension().areno_varlen_causal_attention_forward(
            q.contiguous(), k.contiguous(), v.contiguous(), cu_seqlens.contiguous(), window_left, softmax_scale
        )
        ctx.save_for_backward(q, k, v, out, cu_seqlens)
        ctx.window_left = window_left
        ctx.softmax_scale = softmax_scale
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, out, cu_seqlens = ctx.saved_tensors
        dq, dk, dv = _extension().areno_attention_backward(
            grad_output.contiguous(), q.contiguous(), k.contiguous(), v.contiguous(), out.contiguous(),
            cu_seqlens.contiguous(), None, None, ctx.window_left, ctx.softmax_scale, True,
        )  # fmt: skip
        # (the kernels round their fp32 sums to the inputs' dtype at the store: the casts of the reference's wrapper,
        # ``areno/accel/attention.py:117-118`` there, without fp32 tensors in between)
        return dq, dk, dv, None, None, None


class _PagedDecode(torch.autograd.Function):
    """The decode op under autograd.  As in the reference (``_ArenoPagedCausalAttentionDecode``,
    ``areno/accel/attention.py:212-264`` there) the forward is the kernel and the backward recomputes the attention
    densely in fp32 with tensor ops and lets autograd differentiate that: gradients for ``q`` and for the (unquantized)
    cache tensors as they stand after the append, none for the update rows.  A training-side convenience, not a fast
    path: it gathers every row's pages into one ``(batch, tokens, kv_heads, head_dim)`` tensor."""

    @staticmethod
    def forward(ctx, call, q, k_update, v_update, k_cache, v_cache, k_scale, v_scale, block_table, cache_seqlens,
                window_left, softmax_scale):
        # (k_update / v_update are inputs so that an output whose only differentiable inputs are the update rows stays
        # in the graph; their gradient is None)
        out = call()
        ctx.save_for_backward(q, k_cache, v_cache, k_scale, v_scale, block_table, cache_seqlens)
        ctx.window_left = window_left
        ctx.softmax_scale = softmax_scale
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k_cache, v_cache, k_scale, v_scale, block_table, cache_seqlens = ctx.saved_tensors
        quantized = k_scale is not None
        bs = k_cache.shape[1]
        group = q.shape[1] // k_cache.shape[2]
        lengths = cache_seqlens.long() + 1  # the appended token is visible
        cols = (int(lengths.max()) + bs - 1) // bs
        table = block_table[:, :cols].long().clamp(0, k_cache.shape[0] - 1)  # (columns past a row's length are masked)
        with torch.enable_grad():
            q32 = q.detach().float().requires_grad_(True)
            if quantized:
                k32 = k_cache.float() * k_scale.float().unsqueeze(-1)
                v32 = v_cache.float() * v_scale.float().unsqueeze(-1)
            else:
                k32 = k_cache.detach().float().requires_grad_(True)
                v32 = v_cache.detach().float().requires_grad_(True)
            keys = k32[table].flatten(1, 2).repeat_interleave(group, dim=2)  # (batch, tokens, q heads, head_dim)
            values = v32[table].flatten(1, 2).repeat_interleave(group, dim=2)
            t = torch.arange(keys.shape[1], device=q.device)
            visible = t[None, :] < lengths[:, None]
            if ctx.window_left >= 0:
                visible &= t[None, :] >= (lengths[:, None] - 1 - ctx.window_left)
            # slots no query sees may hold anything (never written, or poisoned): keep them out of the arithmetic
            keys = torch.where(visible[:, :, None, None], keys, 0.0)
            values = torch.where(visible[:, :, None, None], values, 0.0)
            scores = torch.einsum("bhd,bthd->bht", q32, keys) * ctx.softmax_scale
            probs = torch.softmax(scores.masked_fill(~visible[:, None, :], float("-inf")), dim=-1)
            out = torch.einsum("bht,bthd->bhd", probs, values)
            wanted = (q32,) if quantized else (q32, k32, v32)
            grads = torch.autograd.grad(out, wanted, grad_output.float())
        dq = grads[0].to(q.dtype)
        dk, dv = (None, None) if quantized else (grads[1].to(k_cache.dtype), grads[2].to(v_cache.dtype))
        return None, dq, None, None, dk, dv, None, None, None, None, None, None


def _rows_of(x: torch.Tensor) -> torch.Tensor:
    """``(batch, heads, seq, d)`` -> contiguous ``(batch * seq, heads, d)``."""
    b, h, n, d = x.shape
    return x.transpose(1, 2).reshape(b * n, h, d).contiguous()


class _CausalAttention(torch.autograd.Function):
    """Forward and backward of the dense op (``_ArenoCausalAttention``, ``areno/accel/attention.py:78-118`` there).
    The forward is served by the paged prefill kernel: ``k`` / ``v`` are viewed as one page per batch row
    (``block_size = Sk``) and ``query_start`` becomes the cached-context length."""

    @staticmethod
    def forward(ctx, q, k, v, query_start: int, window_left: int, softmax_scale: float):
        batch, heads, sq, d = q.shape
        dev = q.device
        k_pool = k.transpose(1, 2).contiguous()  # (batch, Sk, heads, D): one page per row
        v_pool = v.transpose(1, 2).contiguous()
        table = torch.arange(batch, device=dev, dtype=torch.int32).view(batch, 1)
        cu = torch.arange(batch + 1, device=dev, dtype=torch.int32) * sq
        start = torch.full((batch,), query_start, device=dev, dtype=torch.int32)
        out = _extension().areno_paged_varlen_causal_attention_forward(
            _rows_of(q), k_pool, v_pool, table, cu, start, window_left, softmax_scale, None, None
        )
        out = out.view(batch, sq, heads, d).transpose(1, 2)
        ctx.save_for_backward(q, k, v, out)
        ctx.query_start = query_start
        ctx.window_left = window_left
        ctx.softmax_scale = softmax_scale
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, out = ctx.saved_tensors
        batch, heads, sq, d = q.shape
        sk = k.shape[2]
        dev = q.device
        cu_q = torch.arange(batch + 1, device=dev, dtype=torch.int32) * sq
        cu_k = torch.arange(batch + 1, device=dev, dtype=torch.int32) * sk
        start = torch.full((batch,), ctx.query_start, device=dev, dtype=torch.int32)
        dq, dk, dv = _extension().areno_attention_backward(
            _rows_of(grad_output), _rows_of(q), _rows_of(k), _rows_of(v), _rows_of(out), cu_q, cu_k, start,
            ctx.window_left, ctx.softmax_scale, True,
        )  # fmt: skip
        dq = dq.view(batch, sq, heads, d).transpose(1, 2)
        dk = dk.view(batch, sk, heads, d).transpose(1, 2)
        dv = dv.view(batch, sk, heads, d).transpose(1, 2)
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None, None


_PLAN_DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _decode_in_double(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left, num_splits,
                      softmax_scale):
    """float64 tensors: the reference's kernels read doubles, compute in fp32 and write doubles
    (``AT_DISPATCH_FLOATING_TYPES_AND2`` with float accumulators, ``areno/accel/csrc/attention.cu:979`` there), so
    the op runs on fp32 copies and the result is cast back; the update rows go into the float64 pages as they are."""
    bs, max_blocks = k_cache.shape[1], block_table.shape[1]
    with torch.no_grad():
        pos = cache_seqlens.long()
        col = torch.div(pos, bs, rounding_mode="floor")
        ok = (pos >= 0) & (col < max_blocks)
        blk = block_table.long().gather(1, col.clamp(0, max_blocks - 1).unsqueeze(1)).squeeze(1)
        ok &= (blk >= 0) & (blk < k_cache.shape[0])
        rows = ok.nonzero().squeeze(1)
        k_cache[blk[rows], (pos - col * bs)[rows]] = k_update.detach()[rows]
        v_cache[blk[rows], (pos - col * bs)[rows]] = v_update.detach()[rows]
    out = areno_paged_causal_attention_decode(
        q.float(), k_update.float(), v_update.float(), k_cache.float(), v_cache.float(), block_table, cache_seqlens,
        window_left=window_left, num_splits=num_splits, softmax_scale=_scale(q, softmax_scale),
    )  # fmt: skip
    return out.double()


@torch._dynamo.disable
def areno_paged_decode_plan(
    block_table: torch.Tensor,
    cache_seqlens: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    *,
    q_heads: int,
    q_dtype: torch.dtype = torch.bfloat16,
    window_left: int | None = None,
    with_update: bool = True,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
    prefix_group_rows: int | None = None,
    shared_prefix_lens: torch.Tensor | None = None,
    buffer: torch.Tensor | None = None,
):
    """Build the work list of one decode step once, for all layers of the step.

    ``block_table`` and ``cache_seqlens`` are the same for every layer of a decode step (the reference builds one
    ``InferMeta`` per step, ``areno/engine/inference.py:935`` there), so what the decode kernel derives from them --
    which wave reads which tokens, where it starts and the block ids of its first tile -- is computed by one small
    launch here and handed to every layer's :func:`areno_paged_causal_attention_decode` call as ``plan=``.  The caches
    are any layer's (their shape, dtype and alignment are what matters); ``with_update`` says whether those calls pass
    update rows.  ``buffer`` (optional uint8 CUDA tensor) makes the plan reuse caller memory, e.g. inside a captured
    graph that rebuilds the plan from static tables on every replay.  Legal inside stream capture.
    """
    op = "areno_paged_decode_plan"
    if not _all_on_gpu(block_table, cache_seqlens, k_cache, v_cache, k_scale, v_scale, shared_prefix_lens, buffer):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if block_table.dim() != 2 or cache_seqlens.dim() != 1:
        raise ValueError(f"{op} expects block_table 2D and cache_seqlens 1D")
    if block_table.dtype != torch.int32 or cache_seqlens.dtype != torch.int32:
        raise ValueError(f"{op} expects int32 block_table and cache_seqlens")
    if q_dtype not in _PLAN_DTYPE_CODES:
        raise ValueError(f"{op} expects q_dtype float32, float16 or bfloat16")
    if (prefix_group_rows is None) != (shared_prefix_lens is None):
        raise ValueError(f"{op} expects prefix_group_rows and shared_prefix_lens together")
    _check_scales(op, k_cache, k_scale, v_scale)
    return _extension().areno_paged_decode_plan(
        block_table.contiguous(), cache_seqlens.contiguous(), k_cache, v_cache, k_scale, v_scale,
        _PLAN_DTYPE_CODES[q_dtype], int(q_heads), _window_left(window_left), bool(with_update),
        0 if prefix_group_rows is None else int(prefix_group_rows),
        None if shared_prefix_lens is None else shared_prefix_lens.contiguous(), buffer,
    )  # fmt: skip


@torch._dynamo.disable
def areno_paged_causal_attention_decode(
    q: torch.Tensor,
    k_update: torch.Tensor,
    v_update: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    cache_seqlens: torch.Tensor,
    *,
    window_left: int | None = None,
    num_splits: int = 8,
    softmax_scale: float | None = None,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
    prefix_group_rows: int | None = None,
    shared_prefix_lens: torch.Tensor | None = None,
    plan=None,
) -> torch.Tensor:
    """Apply single-token paged-cache causal attention to ``(batch, heads, dim)`` Q.

    Appends ``k_update``/``v_update`` at position ``cache_seqlens[b]`` of each sequence
    (mutating the caches, and the scale pools for quantized caches, in place), then attends
    over positions ``[0, cache_seqlens[b]]``.  ``num_splits`` is a hint: ``1`` keeps one
    partial per row, any other value lets the kernel pick fixed-size KV chunks.

    ``prefix_group_rows`` / ``shared_prefix_lens`` (optional, together): rows
    ``[i * prefix_group_rows, (i + 1) * prefix_group_rows)`` list the same block ids for their first
    ``shared_prefix_lens[i]`` tokens (the samples of one prompt in a rollout); those pages are then read once for
    several rows instead of once per row.  The result is the same.

    ``plan`` (optional): what :func:`areno_paged_decode_plan` built from the same ``block_table``, ``cache_seqlens``,
    window and prefix groups.  The tables are the same for every layer of a decode step, so one plan serves all of
    them; the result is bit-identical to the call without a plan.
    """
    op = "areno_paged_causal_attention_decode"
    if not _all_on_gpu(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, k_scale, v_scale):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if q.dim() != 3:
        raise ValueError(f"{op} expects q shaped (batch, heads, head_dim)")
    if k_update.dim() != 3 or v_update.dim() != 3:
        raise ValueError(f"{op} expects k/v updates shaped (batch, kv_heads, head_dim)")
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise ValueError(f"{op} expects 4D paged cache tensors")
    if block_table.dim() != 2 or cache_seqlens.dim() != 1:
        raise ValueError(f"{op} expects block_table 2D and cache_seqlens 1D")
    if block_table.dtype != torch.int32 or cache_seqlens.dtype != torch.int32:
        raise ValueError(f"{op} expects int32 block_table and cache_seqlens")
    _check_scales(op, k_cache, k_scale, v_scale)
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        # a contiguous copy would silently drop the in-place cache append
        raise ValueError(f"{op} expects contiguous cache tensors (they are updated in place)")
    if k_scale is not None and not (k_scale.is_contiguous() and v_scale.is_contiguous()):
        raise ValueError(f"{op} expects contiguous scale tensors (they are updated in place)")
    if q.dtype == torch.float64 and k_cache.dtype == torch.float64:
        return _decode_in_double(q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left,
                                 num_splits, softmax_scale)  # fmt: skip
    ext = _extension()
    args = (
        q.contiguous(), k_update.contiguous(), v_update.contiguous(), k_cache, v_cache,
        block_table.contiguous(), cache_seqlens.contiguous(),
        _window_left(window_left), int(num_splits), _scale(q, softmax_scale),
    )  # fmt: skip
    if (prefix_group_rows is None) != (shared_prefix_lens is None):
        raise ValueError(f"{op} expects prefix_group_rows and shared_prefix_lens together")
    if shared_prefix_lens is not None:
        if not shared_prefix_lens.is_cuda:
            raise RuntimeError(f"{op} requires CUDA tensors")
        if int(prefix_group_rows) < 1 or q.shape[0] % int(prefix_group_rows) != 0:
            raise ValueError(f"{op} expects the batch to be a multiple of prefix_group_rows")
        if shared_prefix_lens.dtype != torch.int32 or shared_prefix_lens.shape != (q.shape[0] // int(prefix_group_rows),):
            raise ValueError(f"{op} expects int32 shared_prefix_lens shaped (batch / prefix_group_rows,)")
        groups = (int(prefix_group_rows), shared_prefix_lens.contiguous())
    else:
        groups = (0, None)
    if plan is not None:

        def call():
            return ext.areno_paged_causal_attention_decode_forward_planned(*args, k_scale, v_scale, *groups, plan)
    elif shared_prefix_lens is not None:

        def call():
            return ext.areno_paged_causal_attention_decode_forward_scaled(*args, k_scale, v_scale, *groups)
    elif k_scale is None:

        def call():
            return ext.areno_paged_causal_attention_decode_forward(*args)
    else:

        def call():
            return ext.areno_paged_causal_attention_decode_forward_scaled(*args, k_scale, v_scale, 0, None)

    # the update rows are in the graph like q and the caches (their gradient is None, as in the reference: the
    # output reaches them only through the in-place cache write, which autograd does not see)
    differentiable = (q, k_update, v_update, k_cache, v_cache) if k_scale is None else (q, k_update, v_update)
    if torch.is_grad_enabled() and any(t.requires_grad for t in differentiable):
        return _PagedDecode.apply(call, q, k_update, v_update, k_cache, v_cache, k_scale, v_scale, block_table,
                                  cache_seqlens, _window_left(window_left), _scale(q, softmax_scale))  # fmt: skip
    return call()


@torch._dynamo.disable
def areno_varlen_causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    *,
    window_left: int | None = None,
    softmax_scale: float | None = None,
) -> torch.Tensor:
    """Apply packed causal attention to flat ``(tokens, heads, head_dim)`` tensors."""
    op = "areno_varlen_causal_attention"
    if not _all_on_gpu(q, k, v, cu_seqlens):
        raise RuntimeError(f"{op} requires CUDA q, k, v, and cu_seqlens tensors")
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError(f"{op} expects q/k/v tensors shaped (tokens, heads, head_dim)")
    if cu_seqlens.dim() != 1 or cu_seqlens.dtype != torch.int32:
        raise ValueError(f"{op} expects an int32 1D cu_seqlens tensor")
    if q.shape[0] != k.shape[0] or q.shape[0] != v.shape[0]:
        raise ValueError(f"{op} token count mismatch")
    if k.shape[1] != v.shape[1] or q.shape[1] % k.shape[1] != 0:
        raise ValueError(f"{op} expects q heads to be divisible by kv heads")
    if q.shape[2] != k.shape[2] or q.shape[2] != v.shape[2]:
        raise ValueError(f"{op} head dim mismatch")
    if q.dtype == torch.float64 and k.dtype == torch.float64 and v.dtype == torch.float64:
        # the reference's kernels read doubles and compute in fp32 (attention.cu:846 there): the same through casts
        return _VarlenCausalAttention.apply(q.float(), k.float(), v.float(), cu_seqlens, _window_left(window_left),
                                            _scale(q, softmax_scale)).double()  # fmt: skip
    return _VarlenCausalAttention.apply(q, k, v, cu_seqlens, _window_left(window_left), _scale(q, softmax_scale))


@torch._dynamo.disable
def areno_causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    query_start: int = 0,
    window_left: int | None = None,
    softmax_scale: float | None = None,
) -> torch.Tensor:
    """Apply causal attention to ``(batch, heads, seqlen, head_dim)`` tensors.

    Served by the paged prefill kernel: ``k``/``v`` are viewed as one page per batch row
    (``block_size = Sk``) and ``query_start`` becomes the cached-context length, so query ``i``
    sits at position ``query_start + i``.  Requires ``Sk >= query_start + Sq`` (every position a
    query may see exists as a key).
    """
    op = "areno_causal_attention"
    if not _all_on_gpu(q, k, v):
        raise RuntimeError(f"{op} requires CUDA q, k, and v tensors")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError(f"{op} expects q/k/v tensors shaped (batch, heads, seqlen, head_dim)")
    if q.shape[0] != k.shape[0] or q.shape[0] != v.shape[0]:
        raise ValueError(f"{op} batch size mismatch")
    if q.shape[1] != k.shape[1] or q.shape[1] != v.shape[1]:
        raise ValueError(f"{op} head count mismatch")
    if q.shape[-1] != k.shape[-1] or q.shape[-1] != v.shape[-1]:
        raise ValueError(f"{op} head dim mismatch")
    sk = k.shape[2]
    if sk < int(query_start) + q.shape[2]:
        raise ValueError(f"{op} needs at least query_start + q_len = {int(query_start) + q.shape[2]} keys, got {sk}")
    if q.dtype == torch.float64 and k.dtype == torch.float64 and v.dtype == torch.float64:
        return _CausalAttention.apply(q.float(), k.float(), v.float(), int(query_start), _window_left(window_left),
                                      _scale(q, softmax_scale)).double()  # fmt: skip
    return _CausalAttention.apply(q, k, v, int(query_start), _window_left(window_left), _scale(q, softmax_scale))


@torch._dynamo.disable
def areno_paged_cache_write(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cache_block_ids: torch.Tensor,
    cache_block_offsets: torch.Tensor,
    *,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
) -> None:
    """Store packed ``(tokens, kv_heads, head_dim)`` K/V at ``cache[ids[t], offsets[t]]``, quantizing on the way.

    For ``int8`` / ``float8_e4m3fn`` caches each ``(token, kv head)`` row gets its own scale,
    written to ``k_scale``/``v_scale`` at the same ``(block, slot)``.
    """
    op = "areno_paged_cache_write"
    if not _all_on_gpu(k, v, k_cache, v_cache, cache_block_ids, cache_block_offsets, k_scale, v_scale):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if k.dim() != 3 or v.dim() != 3:
        raise ValueError(f"{op} expects k/v shaped (tokens, kv_heads, head_dim)")
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise ValueError(f"{op} expects 4D paged cache tensors")
    if cache_block_ids.dim() != 1 or cache_block_offsets.dim() != 1:
        raise ValueError(f"{op} expects 1D cache_block_ids and cache_block_offsets")
    if cache_block_ids.dtype != torch.int64 or cache_block_offsets.dtype != torch.int64:
        raise ValueError(f"{op} expects int64 cache_block_ids and cache_block_offsets")
    _check_scales(op, k_cache, k_scale, v_scale)
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError(f"{op} expects contiguous cache tensors (they are updated in place)")
    if k_scale is not None and not (k_scale.is_contiguous() and v_scale.is_contiguous()):
        raise ValueError(f"{op} expects contiguous scale tensors (they are updated in place)")
    _extension().areno_paged_cache_write(
        k.contiguous(), v.contiguous(), k_cache, v_cache,
        cache_block_ids.contiguous(), cache_block_offsets.contiguous(), k_scale, v_scale,
    )  # fmt: skip


@torch._dynamo.disable
def areno_paged_varlen_causal_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    context_lens: torch.Tensor,
    *,
    window_left: int | None = None,
    softmax_scale: float | None = None,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
) -> torch.Tensor:
    """Causal attention of packed new queries ``(tokens, heads, head_dim)`` over paged KV.

    The new tokens' K/V must already be in the cache.  Query ``i`` of sequence ``s`` sits at
    absolute position ``context_lens[s] + i`` and sees keys ``[0, context_lens[s] + i]``.
    """
    op = "areno_paged_varlen_causal_attention"
    _no_autograd(op, q)
    if not _all_on_gpu(q, k_cache, v_cache, block_table, cu_seqlens_q, context_lens, k_scale, v_scale):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if q.dim() != 3:
        raise ValueError(f"{op} expects q shaped (tokens, heads, head_dim)")
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise ValueError(f"{op} expects 4D paged cache tensors")
    if block_table.dim() != 2 or cu_seqlens_q.dim() != 1 or context_lens.dim() != 1:
        raise ValueError(f"{op} expects block_table 2D, cu_seqlens_q 1D and context_lens 1D")
    if any(t.dtype != torch.int32 for t in (block_table, cu_seqlens_q, context_lens)):
        raise ValueError(f"{op} expects int32 block_table, cu_seqlens_q and context_lens")
    _check_scales(op, k_cache, k_scale, v_scale)
    return _extension().areno_paged_varlen_causal_attention_forward(
        q.contiguous(), k_cache.contiguous(), v_cache.contiguous(), block_table.contiguous(),
        cu_seqlens_q.contiguous(), context_lens.contiguous(), _window_left(window_left), _scale(q, softmax_scale),
        _contig(k_scale), _contig(v_scale),
    )  # fmt: skip


@torch._dynamo.disable
def areno_qk_norm_rope_cache_write(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    position_ids: torch.Tensor,
    cos_cached: torch.Tensor,
    sin_cached: torch.Tensor,
    *,
    q_norm_weight: torch.Tensor | None = None,
    k_norm_weight: torch.Tensor | None = None,
    eps: float = 1e-6,
    k_cache: torch.Tensor | None = None,
    v_cache: torch.Tensor | None = None,
    cache_block_ids: torch.Tensor | None = None,
    cache_block_offsets: torch.Tensor | None = None,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
    rope_rows: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The layer's steps in front of attention in one kernel: ``q_norm`` / ``k_norm`` (per-head RMSNorm, fp32
    weights), rotary embedding from the ``(max_position, head_dim)`` float32 tables of ``RotaryEmbedding``, and,
    when caches are given, the quantizing scatter of the new K/V rows to ``cache[ids[t], offsets[t]]``.

    ``q (T, Hq, D)``, ``k`` / ``v (T, Hkv, D)`` fp16 or bf16; returns ``(q, k)`` after norm and rotary.  The pages
    receive exactly what ``areno_paged_cache_write(k_out, v, ...)`` would store.

    ``rope_rows``: what :func:`areno_rope_rows` made of ``position_ids`` and the tables for this dtype, once per step
    for all layers; the kernel then reads a token's prepared cosines and sines instead of fetching its position and
    table rows and rounding them for every (token, head) row.  Same results, bit for bit; ``position_ids`` and the
    tables are not looked at.
    """
    op = "areno_qk_norm_rope_cache_write"
    tensors = (q, k, v, position_ids, cos_cached, sin_cached, q_norm_weight, k_norm_weight, k_cache, v_cache,
               cache_block_ids, cache_block_offsets, k_scale, v_scale, rope_rows)  # fmt: skip
    if not _all_on_gpu(*tensors):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError(f"{op} expects q/k/v shaped (tokens, heads, head_dim)")
    if q.dtype not in (torch.float16, torch.bfloat16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError(f"{op} expects fp16 or bf16 q/k/v of one dtype")
    if (k_cache is None) != (v_cache is None):
        raise ValueError(f"{op} expects k_cache and v_cache together")
    if k_cache is not None:
        if cache_block_ids is None or cache_block_offsets is None:
            raise ValueError(f"{op} expects cache_block_ids and cache_block_offsets with the caches")
        _check_scales(op, k_cache, k_scale, v_scale)
        if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
            raise ValueError(f"{op} expects contiguous cache tensors (they are updated in place)")
    weights = (None if q_norm_weight is None else q_norm_weight.to(torch.float32).contiguous(),
               None if k_norm_weight is None else k_norm_weight.to(torch.float32).contiguous())  # fmt: skip
    if rope_rows is not None:
        if rope_rows.dtype != torch.float32 or rope_rows.shape != (q.shape[0], 2, q.shape[2]):
            raise ValueError(f"{op} expects rope_rows from areno_rope_rows for these tokens: float32 (tokens, 2, head_dim)")
        return tuple(_extension().areno_qk_norm_rope_cache_write_rows(
            q.contiguous(), k.contiguous(), v.contiguous(), rope_rows.contiguous(), *weights, float(eps), k_cache, v_cache,
            _contig(cache_block_ids), _contig(cache_block_offsets), k_scale, v_scale,
        ))  # fmt: skip
    q_out, k_out = _extension().areno_qk_norm_rope_cache_write(
        q.contiguous(), k.contiguous(), v.contiguous(), position_ids.reshape(-1).to(torch.int64).contiguous(),
        cos_cached.to(torch.float32).contiguous(), sin_cached.to(torch.float32).contiguous(), *weights,
        float(eps), k_cache, v_cache, _contig(cache_block_ids), _contig(cache_block_offsets), k_scale, v_scale,
    )  # fmt: skip
    return q_out, k_out


def areno_rope_rows(position_ids: torch.Tensor, cos_cached: torch.Tensor, sin_cached: torch.Tensor,
                    dtype: torch.dtype) -> torch.Tensor:  # fmt: skip
    """The rotary rows of a step's tokens for activations of ``dtype`` (fp16 / bf16): float32 ``(tokens, 2, head_dim)``,
    row ``t`` holding ``cos_cached[position_ids[t]]`` cast to ``dtype`` and ``sin_cached[position_ids[t]]`` cast to
    ``dtype`` with rotate_half's sign (minus on the first half of the head).  ``position_ids`` are the same for every
    layer of a step (``layers/attention.py:94-96`` in the reference hands one tensor down), so this runs once per step
    and every layer's :func:`areno_qk_norm_rope_cache_write` takes the result as ``rope_rows``."""
    op = "areno_rope_rows"
    if not _all_on_gpu(position_ids, cos_cached, sin_cached):
        raise RuntimeError(f"{op} requires CUDA tensors")
    if dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"{op} expects an fp16 or bf16 activation dtype")
    like = torch.empty(0, dtype=dtype, device=position_ids.device)
    return _extension().areno_rope_rows(position_ids.reshape(-1).to(torch.int64).contiguous(),
                                        cos_cached.to(torch.float32).contiguous(),
                                        sin_cached.to(torch.float32).contiguous(), like)  # fmt: skip
