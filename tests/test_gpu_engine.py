"""The backend module driven the way the engine drives it: prompt prefill (store + attention), a second prefill
chunk that must see the first, then decode steps, on plain and quantized caches; every output against the CPU oracle
on the (dequantized) cache contents."""

import pytest
import torch

from areno_amd.engine import InferMeta, allocate_kv_caches, build_infer_attention_backend
from oracle import attention_ref as ar
from tests.gpu_util import DEV, assert_close, dequant_cpu, tolerances

pytestmark = pytest.mark.gpu

BS = 16


def _block_plan(total_lens, num_blocks, gen):
    """Shuffled pages for each sequence, enough for ``total_lens`` tokens; returns the int32 block table."""
    perm = torch.randperm(num_blocks - 1, generator=gen).tolist()  # the last block stays free as the scratch block
    need = [(n + BS - 1) // BS for n in total_lens]
    table = torch.full((len(total_lens), max(need)), num_blocks - 1, dtype=torch.int32)
    for s, n in enumerate(need):
        table[s, :n] = torch.tensor([perm.pop() for _ in range(n)], dtype=torch.int32)
    return table


def _write_plan(table, starts, counts):
    ids, offs = [], []
    for s, (a, n) in enumerate(zip(starts, counts)):
        pos = torch.arange(a, a + n)
        ids.append(table[s].long()[pos // BS])
        offs.append(pos % BS)
    return torch.cat(ids), torch.cat(offs)


@pytest.mark.parametrize("kv,hq,hkv,d,dv", [("auto", 8, 2, 64, 64), ("int8", 28, 4, 128, 128), ("fp8", 8, 8, 128, 96)])
def test_prefill_chunk_decode_loop(kv, hq, hkv, d, dv):
    gen = torch.Generator().manual_seed(41)
    dtype = torch.bfloat16
    prompt, chunk2, steps = [37, 5, 64], [3, 10, 1], 3
    total = [a + b + steps for a, b in zip(prompt, chunk2)]
    num_blocks = sum((n + BS - 1) // BS for n in total) + 4
    layer = allocate_kv_caches(1, num_blocks, BS, hkv, d, DEV, dtype, kv)[0]
    table = _block_plan(total, num_blocks, gen)
    backend = build_infer_attention_backend()
    name = {"auto": "bf16"}.get(kv, kv)
    scale = d**-0.5

    def rand(t, h, w):
        return torch.randn(1, t, h, w, generator=gen).to(dtype)

    def call(q, k, v, meta):
        return backend(q.to(DEV), k.to(DEV), v.to(DEV), layer.k_cache, layer.v_cache, meta, softmax_scale=scale,
                       k_scale=layer.k_scale, v_scale=layer.v_scale)  # fmt: skip

    def cache_cpu():
        return dequant_cpu(layer.k_cache, layer.k_scale), dequant_cpu(layer.v_cache, layer.v_scale)

    # ---- prompt prefill: attention over the fresh (unquantized) K/V, pages written on the side ------------------
    t1 = sum(prompt)
    q, k, v = rand(t1, hq, d), rand(t1, hkv, d), rand(t1, hkv, dv)
    cu = torch.tensor([0] + list(torch.tensor(prompt).cumsum(0)), dtype=torch.int32)
    ids, offs = _write_plan(table, [0, 0, 0], prompt)
    meta = InferMeta(mode="prefill", cu_seqlens=cu.to(DEV), max_seqlen=max(prompt), block_table=table.to(DEV),
                     cache_block_ids=ids.to(DEV), cache_block_offsets=offs.to(DEV))  # fmt: skip
    out = call(q, k, v, meta)
    assert out.shape == (1, t1, hq, dv)
    v_pad = torch.nn.functional.pad(v[0].float(), (0, d - dv))
    want = ar.ref_varlen(q[0].float(), k[0].float(), v_pad, cu, -1, scale)[..., :dv]
    assert_close(out[0], want, *tolerances("bf16"), what="prompt prefill")

    # ---- second chunk: must see the cached prompt through the pages -------------------------------------------------
    t2 = sum(chunk2)
    q, k, v = rand(t2, hq, d), rand(t2, hkv, d), rand(t2, hkv, dv)
    cu2 = torch.tensor([0] + list(torch.tensor(chunk2).cumsum(0)), dtype=torch.int32)
    ids, offs = _write_plan(table, prompt, chunk2)
    ctx = torch.tensor(prompt, dtype=torch.int32)
    meta = InferMeta(mode="prefill", cu_seqlens=cu2.to(DEV), max_seqlen=max(chunk2), block_table=table.to(DEV),
                     cache_block_ids=ids.to(DEV), cache_block_offsets=offs.to(DEV), context_lens=ctx.to(DEV))  # fmt: skip
    out = call(q, k, v, meta)
    kc, vc = cache_cpu()
    want = ar.ref_paged_varlen_prefill(q[0].float(), kc, vc, table, cu2, ctx, -1, scale)[..., :dv]
    assert_close(out[0], want, *tolerances(name), what="chunk over cached context")

    # ---- decode steps ---------------------------------------------------------------------------------------------------
    lens = torch.tensor([a + b for a, b in zip(prompt, chunk2)], dtype=torch.int32)
    for step in range(steps):
        q, k, v = rand(3, hq, d), rand(3, hkv, d), rand(3, hkv, dv)
        meta = InferMeta(mode="decode", cache_seqlens=(lens + step).to(DEV), block_table=table.to(DEV))
        out = call(q, k, v, meta)
        assert out.shape == (1, 3, hq, dv)
        kc, vc = cache_cpu()
        want = ar.ref_paged_decode(q[0].float(), kc, vc, table, lens + step, -1, scale)[..., :dv]
        assert_close(out[0], want, *tolerances(name), what=f"decode step {step}")


def test_loop_driven_by_device_block_tables():
    """Same loop with the page bookkeeping on the device: tables, write slots and positions come from
    DeviceBlockTables (no host-built table is uploaded), decode crosses page borders, one sequence finishes and a
    new one is admitted into the freed pages; outputs against the oracle reading through the device's own table."""
    from areno_amd.engine import DeviceBlockTables
    from oracle.block_table_ref import RefBlockTables

    gen = torch.Generator().manual_seed(43)
    dtype, hq, hkv, d = torch.bfloat16, 8, 2, 64
    scale = d**-0.5
    num_blocks, max_rows, max_blocks = 12, 4, 6
    layer = allocate_kv_caches(1, num_blocks + 1, BS, hkv, d, DEV, dtype, "int8")[0]
    pages = DeviceBlockTables(num_blocks, max_rows, max_blocks, BS, DEV)
    lists = RefBlockTables(num_blocks, max_rows, max_blocks, BS)  # the reference's host lists, kept in step
    backend = build_infer_attention_backend()

    def same_pages():
        for row in range(max_rows):
            assert pages.row_pages(row) == lists.row_pages(row), f"row {row}"
        assert pages.free_list() == lists.free_list() and pages.status() == (0, -1)

    def rand(t, h):
        return torch.randn(1, t, h, d, generator=gen).to(dtype)

    def call(q, k, v, meta):
        return backend(q.to(DEV), k.to(DEV), v.to(DEV), layer.k_cache, layer.v_cache, meta, softmax_scale=scale,
                       k_scale=layer.k_scale, v_scale=layer.v_scale)  # fmt: skip

    def prefill(rows, lens):
        pages.reserve(rows, lens)
        lists.reserve(rows, lens)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        t = int(cu[-1])
        ids, offs, pos = pages.prefill_slots(rows, [0] * len(rows), cu, t)
        assert pos.cpu().tolist() == [p for n in lens for p in range(n)]
        table = pages.block_table(rows)
        q, k, v = rand(t, hq), rand(t, hkv), rand(t, hkv)
        meta = InferMeta(mode="prefill", cu_seqlens=cu.to(DEV), max_seqlen=max(lens), block_table=table,
                         cache_block_ids=ids, cache_block_offsets=offs)  # fmt: skip
        out = call(q, k, v, meta)
        want = ar.ref_varlen(q[0].float(), k[0].float(), v[0].float(), cu, -1, scale)
        assert_close(out[0], want, *tolerances("bf16"), what="prefill")

    def decode(rows, lens_dev, steps):
        rows_dev = torch.tensor(rows, device=DEV)
        for step in range(steps):
            pages.ensure_decode(rows_dev, lens_dev)
            lists.ensure_decode(rows, lens_dev.cpu().tolist())
            table = pages.block_table(rows_dev)
            assert table.cpu().tolist() == lists.gather(rows, False)
            q, k, v = rand(len(rows), hq), rand(len(rows), hkv), rand(len(rows), hkv)
            meta = InferMeta(mode="decode", cache_seqlens=lens_dev, block_table=table)
            out = call(q, k, v, meta)
            kc, vc = dequant_cpu(layer.k_cache, layer.k_scale), dequant_cpu(layer.v_cache, layer.v_scale)
            want = ar.ref_paged_decode(q[0].float(), kc, vc, table.cpu(), lens_dev.cpu(), -1, scale)
            assert_close(out[0], want, *tolerances("int8"), what=f"decode step {step}")
            lens_dev += 1
        pages.check()

    prefill([2, 0, 3], [30, 16, 5])
    lens_dev = torch.tensor([30, 16, 5], dtype=torch.int32, device=DEV)
    decode([2, 0, 3], lens_dev, 4)  # row 0 opens its second page at position 16, row 2 its third at 32
    assert pages.row_pages(2) == [0, 1, 5] and pages.row_pages(0) == [2, 4] and pages.row_pages(3) == [3]
    same_pages()
    pages.release([0])
    lists.release([0])
    prefill([1], [40])  # takes pages 6 .. 8 from the head of the free list; row 0's pages wait at the tail
    assert pages.row_pages(1) == [6, 7, 8] and pages.free_list() == [9, 10, 11, 2, 4]
    lens_dev = torch.tensor([34, 40, 9], dtype=torch.int32, device=DEV)
    decode([2, 1, 3], lens_dev, 9)  # row 3 reaches position 16 one step before row 1 reaches 48
    assert pages.row_pages(1) == [6, 7, 8, 10] and pages.row_pages(3) == [3, 9]
    same_pages()
