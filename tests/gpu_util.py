"""Helpers shared by the GPU parity tests (imported only by tests)."""

from __future__ import annotations

import torch

from areno_amd import workloads
from areno_amd.accel import attention as ops
from oracle import attention_ref as ar
from oracle import quant_ref as qr

DEV = "cuda:0"
BF16_MAX_ABS, BF16_MEAN_ABS = 2e-2, 2e-3  # bf16 / fp16 / fp32 KV vs the fp32 reference
QUANT_MAX_ABS = 5e-2  # int8 / fp8 KV vs the same reference on the dequantized cache


def gpu_quantize(x: torch.Tensor, cache_dtype: torch.dtype):
    """Quantize ``x (N, Hkv, D)`` with the HIP cache-write kernel (one page per token)."""
    n, hkv, d = x.shape
    sdt = torch.float16 if cache_dtype == torch.int8 else torch.float32
    kc = torch.empty((n, 1, hkv, d), dtype=cache_dtype, device=x.device)
    vc = torch.empty_like(kc)
    ks = torch.empty((n, 1, hkv), dtype=sdt, device=x.device)
    vs = torch.empty_like(ks)
    ids = torch.arange(n, device=x.device, dtype=torch.int64)
    ops.areno_paged_cache_write(x, x, kc, vc, ids, torch.zeros_like(ids), k_scale=ks, v_scale=vs)
    return kc.view(n, hkv, d), ks.view(n, hkv)


def dequant_cpu(cache: torch.Tensor, scale: torch.Tensor | None) -> torch.Tensor:
    c = cache.cpu()
    if scale is None:
        return c.float()
    out = qr.dequantize(c, scale.cpu())
    # poisoned (never-read) slots carry NaN scales; keep them NaN so a stray read shows up
    return out


def build_plan(w: workloads.DecodeWorkload, *, window_left=None, grouped=False, buffer=None):
    """The per-step plan of the decode op for a workload's tables."""
    groups = {}
    if grouped:
        groups = dict(prefix_group_rows=w.meta["prefix_group_rows"], shared_prefix_lens=w.meta["shared_prefix_lens"])
    return ops.areno_paged_decode_plan(
        w.block_table, w.cache_seqlens, w.k_cache, w.v_cache, q_heads=w.q.shape[1], q_dtype=w.q.dtype,
        window_left=window_left, k_scale=w.k_scale, v_scale=w.v_scale, buffer=buffer, **groups,
    )  # fmt: skip


def run_decode(w: workloads.DecodeWorkload, *, window_left=None, num_splits=8, planned=False):
    """The decode op on a workload; ``planned`` runs it with a per-step plan built from the same tables."""
    plan = build_plan(w, window_left=window_left) if planned else None
    return ops.areno_paged_causal_attention_decode(
        w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table, w.cache_seqlens,
        window_left=window_left, num_splits=num_splits, softmax_scale=w.softmax_scale,
        k_scale=w.k_scale, v_scale=w.v_scale, plan=plan,
    )  # fmt: skip


def expected_decode(w: workloads.DecodeWorkload, *, window_left=None, rows=None):
    """Oracle on the post-step cache (dequantized for int8/fp8), optionally on a subset of rows."""
    kc = dequant_cpu(w.k_cache, w.k_scale)
    vc = dequant_cpu(w.v_cache, w.v_scale)
    q, table, lens = w.q.cpu().float(), w.block_table.cpu(), w.cache_seqlens.cpu()
    if rows is not None:
        q, table, lens = q[rows], table[rows], lens[rows]
    return ar.ref_paged_decode(q, kc, vc, table, lens, ar.window_left_arg(window_left), w.softmax_scale)


def assert_close(got: torch.Tensor, want: torch.Tensor, max_abs: float, mean_abs: float | None = None, what=""):
    got = got.detach().cpu().float()
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want.float()).abs()
    assert err.max().item() <= max_abs, f"{what}: max-abs {err.max().item():.4g} > {max_abs}"
    if mean_abs is not None:
        assert err.mean().item() <= mean_abs, f"{what}: mean-abs {err.mean().item():.4g} > {mean_abs}"
    return err.max().item(), err.mean().item()


def tolerances(kv: str):
    return (QUANT_MAX_ABS, None) if kv in ("int8", "fp8") else (BF16_MAX_ABS, BF16_MEAN_ABS)


def compact_pages(cache, scale, table_rows: torch.Tensor):
    """The pages that ``table_rows`` (CPU int tensor, any shape) names, dequantized on the CPU, and the same table with the ids
    renumbered into that compact pool: the oracle then works on a pool of a few hundred MB instead of the whole cache."""
    ids, inverse = torch.unique(table_rows.long().flatten(), return_inverse=True)
    pages = cache[ids.to(cache.device)].cpu()
    sc = None if scale is None else scale[ids.to(scale.device)].cpu()
    dense = pages.float() if sc is None else qr.dequantize(pages, sc)
    return dense, inverse.view(table_rows.shape).to(torch.int32)


def expected_decode_rows(w: workloads.DecodeWorkload, rows, *, window_left=None):
    """Oracle on the post-step cache for the rows in ``rows`` (a list of row indices), touching only the pages those rows read."""
    rows = torch.as_tensor(rows, dtype=torch.long)
    bs = w.k_cache.shape[1]
    lens = w.cache_seqlens.cpu()[rows]
    table = w.block_table.cpu()[rows]
    # columns past a row's last page repeat a valid id (padding): the compact pool keeps them, the oracle never reads them
    cols = int((int(lens.max()) + bs) // bs)
    table = table[:, :cols]
    kc, compact = compact_pages(w.k_cache, w.k_scale, table)
    vc, _ = compact_pages(w.v_cache, w.v_scale, table)
    return ar.ref_paged_decode(w.q[rows.to(w.q.device)].cpu().float(), kc, vc, compact, lens,
                               ar.window_left_arg(window_left), w.softmax_scale)  # fmt: skip
