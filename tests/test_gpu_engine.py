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
