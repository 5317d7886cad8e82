"""Seeded synthetic inputs for the five benchmark configurations of the paged attention path.

Shared by the parity tests and ``bench.py`` so both see identical tensors.  Integer
draws (lengths, block permutations) always come from a CPU ``torch.Generator`` and are
therefore identical on every machine; bulk tensor contents are drawn on the target device.

Shapes follow the engine's contracts: caches ``[NB, bs, Hkv, D]``
(``areno/models/qwen3/model.py:309-333`` in the reference), scales ``[NB, bs, Hkv]``,
``block_table (B, MB) int32`` right-padded with the row's last valid id
(``areno/engine/data/rollout_state.py:282-285``), ``cache_seqlens (B,) int32`` = tokens
already cached before the step (``areno/engine/runtime/metadata.py:29-45``).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Callable

import torch

CACHE_DTYPES = {
    "fp32": torch.float32,
    "bf16": torch.bfloat16,
    "fp16": torch.float16,
    "int8": torch.int8,
    "fp8": torch.float8_e4m3fn,
}
SCALE_DTYPES = {"int8": torch.float16, "fp8": torch.float32}

# (codes, scales) = quantize_fn(x (N, Hkv, D), cache_dtype)
QuantizeFn = Callable[[torch.Tensor, torch.dtype], tuple[torch.Tensor, torch.Tensor]]


@dataclass
class DecodeWorkload:
    name: str
    kv: str
    q: torch.Tensor
    k_update: torch.Tensor
    v_update: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    k_scale: torch.Tensor | None
    v_scale: torch.Tensor | None
    block_table: torch.Tensor
    cache_seqlens: torch.Tensor
    softmax_scale: float
    unique_tokens: int  # distinct cached positions read by the step (shared prefix pages counted once)
    logical_tokens: int  # sum over sequences of (L_b + 1)
    meta: dict = field(default_factory=dict)

    @property
    def shape(self) -> tuple[int, int, int, int, int]:
        return (self.q.shape[0], self.q.shape[1], self.k_cache.shape[2], self.q.shape[2], self.k_cache.shape[1])

    def algorithmic_bytes(self) -> int:
        """Compulsory HBM bytes of one decode step: KV (+scales) once per KV head, Q in, out, table ids."""
        b, hq, hkv, d, bs = self.shape
        e = self.k_cache.element_size()
        s = 0 if self.k_scale is None else self.k_scale.element_size()
        kv_bytes = self.unique_tokens * hkv * (2 * d * e + 2 * s)
        lens = self.cache_seqlens.long().cpu() + 1
        ids = int(torch.div(lens + bs - 1, bs, rounding_mode="floor").sum())
        return kv_bytes + 2 * b * hq * d * self.q.element_size() + 4 * ids + 4 * b


@dataclass
class PrefillWorkload:
    name: str
    kv: str
    q: torch.Tensor  # (T, Hq, D)
    k_new: torch.Tensor  # (T, Hkv, D) new tokens' K (already written into the cache too)
    v_new: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    k_scale: torch.Tensor | None
    v_scale: torch.Tensor | None
    block_table: torch.Tensor
    cu_seqlens_q: torch.Tensor
    context_lens: torch.Tensor
    cache_block_ids: torch.Tensor
    cache_block_offsets: torch.Tensor
    softmax_scale: float
    meta: dict = field(default_factory=dict)

    def flops(self) -> int:
        """QK^T + PV with the causal triangle counted exactly: sum 4*Hq*D*n*(ctx + (n+1)/2)."""
        hq, d = self.q.shape[1], self.q.shape[2]
        cu = self.cu_seqlens_q.long().cpu()
        n = cu[1:] - cu[:-1]
        ctx = self.context_lens.long().cpu()
        return int((4 * hq * d * (n * ctx + n * (n + 1) // 2)).sum())


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _randint(g: torch.Generator, lo: int, hi: int, n: int) -> torch.Tensor:
    """``n`` integers uniform in the closed range ``[lo, hi]``."""
    return torch.randint(lo, hi + 1, (n,), generator=g, dtype=torch.int64)


def _assign_blocks(per_seq_blocks: list[list[int]], pool_blocks: int, g: torch.Generator, table_cols: int = 0):
    """Map logical block numbers (0..U-1, shared numbers = shared pages) to a shuffled pool.

    Returns ``(block_table int32 (B, MB), used_ids int64 (U,))``.
    """
    unique = 1 + max(max(r) for r in per_seq_blocks)
    assert pool_blocks >= unique
    perm = torch.randperm(pool_blocks, generator=g)[:unique]
    width = max(max(len(r) for r in per_seq_blocks), table_cols)
    table = torch.empty((len(per_seq_blocks), width), dtype=torch.int32)
    for i, row in enumerate(per_seq_blocks):
        ids = perm[torch.tensor(row, dtype=torch.int64)].to(torch.int32)
        table[i, : len(row)] = ids
        table[i, len(row) :] = ids[-1]  # eager padding: the row's last valid id
    return table, perm


def _values(shape, device, g_dev: torch.Generator, *, std: float = 1.0, outlier_frac: float = 0.0, outlier_mul: float = 8.0):
    x = torch.randn(shape, device=device, generator=g_dev, dtype=torch.float32) * std
    if outlier_frac > 0:
        mask = torch.rand(shape, device=device, generator=g_dev) < outlier_frac
        x = torch.where(mask, x * outlier_mul, x)
    return x


def _fill_caches(
    kv: str,
    nb: int,
    bs: int,
    hkv: int,
    d: int,
    device,
    g_dev: torch.Generator,
    value_dtype: torch.dtype,
    quantize_fn: QuantizeFn | None,
    std: float,
    outlier_frac: float,
    chunk_blocks: int = 4096,
):
    """Allocate and fill K/V pools (+scales for quantized kinds) with random finite data."""
    cdt = CACHE_DTYPES[kv]
    quantized = kv in SCALE_DTYPES
    if quantized and quantize_fn is None:
        raise ValueError("a quantize_fn is required to fill an int8/fp8 cache")
    caches, scales = [], []
    for _ in range(2):
        cache = torch.empty((nb, bs, hkv, d), dtype=cdt, device=device)
        scale = torch.empty((nb, bs, hkv), dtype=SCALE_DTYPES[kv], device=device) if quantized else None
        for lo in range(0, nb, chunk_blocks):
            hi = min(nb, lo + chunk_blocks)
            x = _values((hi - lo, bs, hkv, d), device, g_dev, std=std, outlier_frac=outlier_frac).to(value_dtype)
            if quantized:
                codes, sc = quantize_fn(x.view(-1, hkv, d), cdt)
                cache[lo:hi].view(torch.uint8).copy_(codes.view(torch.uint8).view(hi - lo, bs, hkv, d))
                scale[lo:hi].copy_(sc.view(hi - lo, bs, hkv))
            else:
                cache[lo:hi].copy_(x)
        caches.append(cache)
        scales.append(scale)
    return caches[0], caches[1], scales[0], scales[1]


def poison_unused_slots(w: DecodeWorkload) -> None:
    """Overwrite every cache slot the step must not read (positions > L_b, unused pages) with poison.

    Floating caches get NaN, quantized caches get NaN scales and extreme codes: if a kernel
    touches them the output shows it.  The slot at position L_b is written by the step itself.
    """
    nb, bs = w.k_cache.shape[0], w.k_cache.shape[1]
    live = torch.zeros((nb, bs), dtype=torch.bool)
    table = w.block_table.cpu().long()
    lens = w.cache_seqlens.cpu().long()
    for b in range(table.shape[0]):
        n = int(lens[b])  # positions [0, n) are live before the step
        full, rem = divmod(n, bs)
        live[table[b, :full]] = True
        if rem:
            live[table[b, full], :rem] = True
    dead = (~live).to(w.k_cache.device)
    for cache, scale in ((w.k_cache, w.k_scale), (w.v_cache, w.v_scale)):
        if scale is None:
            cache[dead] = float("nan")
        else:
            cache.view(torch.uint8)[dead] = 0x7F
            scale[dead] = float("nan")


def make_decode_workload(
    name: str,
    *,
    seed: int,
    batch: int,
    hq: int,
    hkv: int,
    d: int,
    bs: int,
    kv: str,
    lengths: torch.Tensor,
    device="cpu",
    act_dtype: torch.dtype = torch.bfloat16,
    std: float = 1.0,
    outlier_frac: float = 0.0,
    softmax_scale: float | None = None,
    pool_blocks: int | None = None,
    pool_slack: float = 0.10,
    shared_prefix_blocks: list[int] | None = None,
    group_size: int = 1,
    table_cols: int = 0,
    quantize_fn: QuantizeFn | None = None,
    poison: bool = False,
) -> DecodeWorkload:
    """Generic decode workload; ``lengths[b]`` = tokens already cached for row ``b``.

    ``shared_prefix_blocks[p]`` (one per group of ``group_size`` consecutive rows) makes the
    rows of a group share their first pages, as rollout samples of one prompt do.
    """
    g = _gen(seed)
    lengths = lengths.to(torch.int64)
    per_seq: list[list[int]] = []
    next_block = 0
    unique_tokens = 0
    for grp in range(batch // group_size):
        shared = 0 if shared_prefix_blocks is None else int(shared_prefix_blocks[grp])
        shared_ids = list(range(next_block, next_block + shared))
        next_block += shared
        unique_tokens += shared * bs
        for j in range(group_size):
            b = grp * group_size + j
            need = (int(lengths[b]) + 1 + bs - 1) // bs
            assert need > shared or shared == 0
            private = list(range(next_block, next_block + need - shared))
            next_block += need - shared
            per_seq.append(shared_ids + private)
            unique_tokens += int(lengths[b]) + 1 - shared * bs
    nb = pool_blocks if pool_blocks is not None else int(math.ceil(next_block * (1.0 + pool_slack)))
    table, _ = _assign_blocks(per_seq, nb, g, table_cols=table_cols)

    g_dev = torch.Generator(device=device)
    g_dev.manual_seed(seed + 7919)
    value_dtype = act_dtype if kv in SCALE_DTYPES else CACHE_DTYPES[kv]
    k_cache, v_cache, k_scale, v_scale = _fill_caches(
        kv, nb, bs, hkv, d, device, g_dev, value_dtype, quantize_fn, std, outlier_frac
    )
    in_dtype = act_dtype if kv in SCALE_DTYPES else CACHE_DTYPES[kv]
    q = _values((batch, hq, d), device, g_dev, std=std).to(in_dtype)
    k_update = _values((batch, hkv, d), device, g_dev, std=std, outlier_frac=outlier_frac).to(in_dtype)
    v_update = _values((batch, hkv, d), device, g_dev, std=std, outlier_frac=outlier_frac).to(in_dtype)
    w = DecodeWorkload(
        name=name,
        kv=kv,
        q=q,
        k_update=k_update,
        v_update=v_update,
        k_cache=k_cache,
        v_cache=v_cache,
        k_scale=k_scale,
        v_scale=v_scale,
        block_table=table.to(device),
        cache_seqlens=lengths.to(torch.int32).to(device),
        softmax_scale=float(softmax_scale if softmax_scale is not None else d**-0.5),
        unique_tokens=unique_tokens,
        logical_tokens=int((lengths + 1).sum()),
        meta={"seed": seed, "pool_blocks": nb, "used_blocks": next_block},
    )
    if shared_prefix_blocks is not None:
        # what the scheduler knows about the batch: rows per prompt and tokens of each prompt's shared pages
        w.meta["prefix_group_rows"] = int(group_size)
        w.meta["shared_prefix_lens"] = torch.tensor([int(n) * bs for n in shared_prefix_blocks], dtype=torch.int32,
                                                    device=device)  # fmt: skip
    if poison:
        poison_unused_slots(w)
    return w


def cfg0_tiny(kv: str = "fp32", *, device="cpu", seed: int = 1000, **kw) -> DecodeWorkload:
    """Tiny paged decode: B=4, 8 q heads / 2 kv heads, D=64, bs=16, L ~ U{17..300}, 128-block pool."""
    g = _gen(seed + 1)
    lengths = _randint(g, 17, 300, 4)
    return make_decode_workload(
        f"cfg0-tiny-{kv}", seed=seed, batch=4, hq=8, hkv=2, d=64, bs=16, kv=kv, lengths=lengths, device=device,
        std=64**-0.5, softmax_scale=64**-0.5, pool_blocks=128, table_cols=19, **kw,
    )  # fmt: skip


def cfg1_qwen7b(kv: str = "bf16", *, device="cpu", seed: int = 1001, batch: int = 64, ctx_lo=512, ctx_hi=4096, **kw):
    """Qwen2.5-7B-like decode: B=64, 28/4 heads, D=128, bs=16, ctx ~ U{512..4096}; bf16 KV (cfg 1) or int8 (cfg 2)."""
    g = _gen(seed + 1)
    lengths = _randint(g, ctx_lo, ctx_hi, batch)
    outliers = 0.01 if kv in SCALE_DTYPES else 0.0
    return make_decode_workload(
        f"cfg{2 if kv == 'int8' else 1}-qwen7b-{kv}" + ("" if batch == 64 else f"-b{batch}"), seed=seed, batch=batch, hq=28, hkv=4, d=128, bs=16, kv=kv,
        lengths=lengths, device=device, outlier_frac=outliers, table_cols=(ctx_hi + 1 + 15) // 16, **kw,
    )  # fmt: skip


def cfg2_qwen7b_int8(**kw) -> DecodeWorkload:
    return cfg1_qwen7b("int8", seed=kw.pop("seed", 1002), **kw)


def cfg3_lengths(seed: int = 1003, prompts: int = 32, samples: int = 8, prefix_lo=256, prefix_hi=2048, median=1000.0,
                 sigma=1.0, cap=32768):
    """The integer draws of the rollout configuration: ``(prefix (prompts,), lengths (prompts * samples,))``."""
    g = _gen(seed + 1)
    prefix = _randint(g, prefix_lo, prefix_hi, prompts)
    cont = torch.exp(torch.randn(prompts * samples, generator=g) * sigma + math.log(median))
    cont = torch.clamp(cont, max=float(cap)).to(torch.int64)
    return prefix, prefix.repeat_interleave(samples) + cont


def cfg3_rollout(kv: str = "fp8", *, device="cpu", seed: int = 1003, prompts: int = 32, samples: int = 8,
                 prefix_lo=256, prefix_hi=2048, median=1000.0, sigma=1.0, cap=32768, hq: int = 32, hkv: int = 8,
                 **kw) -> DecodeWorkload:  # fmt: skip
    """RL-rollout decode: ``prompts x samples`` rows, samples of a prompt share the prompt's full pages."""
    bs = 16
    prefix, lengths = cfg3_lengths(seed, prompts, samples, prefix_lo, prefix_hi, median, sigma, cap)
    shared = [int(p) // bs for p in prefix]
    return make_decode_workload(
        f"cfg3-rollout-{kv}", seed=seed, batch=prompts * samples, hq=hq, hkv=hkv, d=128, bs=bs, kv=kv, lengths=lengths,
        device=device, shared_prefix_blocks=shared, group_size=samples, **kw,
    )  # fmt: skip


def make_prefill_workload(
    name: str,
    *,
    seed: int,
    new_lens: torch.Tensor,
    ctx_lens: torch.Tensor,
    hq: int,
    hkv: int,
    d: int,
    bs: int,
    kv: str,
    device="cpu",
    act_dtype: torch.dtype = torch.bfloat16,
    std: float = 1.0,
    softmax_scale: float | None = None,
    pool_slack: float = 0.10,
    quantize_fn: QuantizeFn | None = None,
) -> PrefillWorkload:
    """Chunked prefill: ``new_lens[s]`` new queries on top of ``ctx_lens[s]`` cached tokens, all KV paged.

    The new tokens' K/V are part of the generated pool contents at their addresses
    (``cache_block_ids/offsets``, the per-token plan of ``rollout_state.py:160-164``) and are
    also returned un-quantized as ``k_new``/``v_new`` so a test can replay the cache write.
    """
    g = _gen(seed)
    new_lens, ctx_lens = new_lens.to(torch.int64), ctx_lens.to(torch.int64)
    per_seq, next_block = [], 0
    for s in range(len(new_lens)):
        need = max(1, (int(ctx_lens[s] + new_lens[s]) + bs - 1) // bs)
        per_seq.append(list(range(next_block, next_block + need)))
        next_block += need
    nb = int(math.ceil(next_block * (1.0 + pool_slack)))
    table, _ = _assign_blocks(per_seq, nb, g)
    cu = torch.zeros(len(new_lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(new_lens, 0).to(torch.int32)
    ids, offs = [], []
    for s in range(len(new_lens)):
        pos = torch.arange(int(ctx_lens[s]), int(ctx_lens[s] + new_lens[s]))
        ids.append(table[s].long()[pos // bs])
        offs.append(pos % bs)
    ids, offs = torch.cat(ids), torch.cat(offs)

    g_dev = torch.Generator(device=device)
    g_dev.manual_seed(seed + 7919)
    value_dtype = act_dtype if kv in SCALE_DTYPES else CACHE_DTYPES[kv]
    k_cache, v_cache, k_scale, v_scale = _fill_caches(
        kv, nb, bs, hkv, d, device, g_dev, value_dtype, quantize_fn, std, 0.0
    )
    t = int(cu[-1])
    in_dtype = value_dtype
    q = _values((t, hq, d), device, g_dev, std=std).to(in_dtype)
    k_new = _values((t, hkv, d), device, g_dev, std=std).to(in_dtype)
    v_new = _values((t, hkv, d), device, g_dev, std=std).to(in_dtype)
    return PrefillWorkload(
        name=name, kv=kv, q=q, k_new=k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache, k_scale=k_scale,
        v_scale=v_scale, block_table=table.to(device), cu_seqlens_q=cu.to(device),
        context_lens=ctx_lens.to(torch.int32).to(device), cache_block_ids=ids.to(device),
        cache_block_offsets=offs.to(device),
        softmax_scale=float(softmax_scale if softmax_scale is not None else d**-0.5),
        meta={"seed": seed, "pool_blocks": nb, "tokens": t},
    )  # fmt: skip


def cfg4_prefill(kv: str = "fp8", *, device="cpu", seed: int = 1004, seqs: int = 16, new_hi: int = 512,
                 ctx_hi: int = 16384, **kw) -> PrefillWorkload:  # fmt: skip
    """Varlen prefill over paged KV: 16 seqs, n ~ U{1..512} new, ctx ~ U{0..16384}, 32/8 heads, D=128, bs=16."""
    g = _gen(seed + 1)
    new_lens = _randint(g, 1, new_hi, seqs)
    ctx_lens = _randint(g, 0, ctx_hi, seqs)
    return make_prefill_workload(
        f"cfg4-prefill-{kv}", seed=seed, new_lens=new_lens, ctx_lens=ctx_lens, hq=32, hkv=8, d=128, bs=16, kv=kv,
        device=device, **kw,
    )  # fmt: skip
