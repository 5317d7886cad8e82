"""Paged decode op vs the CPU oracle on identical seeded inputs.

Tolerances (from the benchmark contract): bf16/fp16/fp32 KV max-abs 2e-2 and mean-abs 2e-3 against
the fp32 reference; int8/fp8 KV max-abs 5e-2 against the same reference on the dequantized cache.
The fused append is checked bit-exactly and by a snapshot diff of the whole pool.
"""

import pytest
import torch

from areno_amd import workloads
from areno_amd.accel import attention as ops
from oracle import quant_ref as qr
from tests.gpu_util import (DEV, assert_close, build_plan, expected_decode, expected_decode_rows, gpu_quantize,
                            run_decode, tolerances)

pytestmark = pytest.mark.gpu


def _check_append(w, before):
    """Only the (block, slot) of position L_b changed, and it holds the (quantized) update bit-exactly."""
    ids, offs = qr.decode_addresses(w.block_table.cpu(), w.cache_seqlens.cpu(), w.k_cache.shape[1])
    touched = torch.zeros(w.k_cache.shape[:2], dtype=torch.bool)
    touched[ids, offs] = True
    names = ("k_cache", "v_cache", "k_scale", "v_scale")
    for name, old in zip(names, before):
        if old is None:
            continue
        new = getattr(w, name).cpu()
        raw_new = new.view(torch.uint8) if new.dtype == torch.float8_e4m3fn else new
        raw_old = old.view(torch.uint8) if old.dtype == torch.float8_e4m3fn else old
        same = raw_new[~touched] == raw_old[~touched]
        if raw_old.is_floating_point():
            same |= raw_old[~touched].isnan()  # poisoned slots stay poisoned
        assert same.all(), f"{name}: a slot other than the append target changed"
    ku, vu = w.k_update.cpu(), w.v_update.cpu()
    if w.k_scale is None:
        assert torch.equal(w.k_cache.cpu()[ids, offs], ku) and torch.equal(w.v_cache.cpu()[ids, offs], vu)
    else:
        for upd, cache, scale in ((ku, w.k_cache, w.k_scale), (vu, w.v_cache, w.v_scale)):
            codes, sc = qr.quantize(upd, cache.dtype)
            assert torch.equal(cache.cpu()[ids, offs].float(), codes.float())
            assert torch.equal(scale.cpu()[ids, offs], sc)


def _snapshot(w):
    return [None if t is None else t.cpu().clone() for t in (w.k_cache, w.v_cache, w.k_scale, w.v_scale)]


@pytest.mark.parametrize("kv", ["fp32", "bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("window_left", [None, 40, 0])
@pytest.mark.parametrize("planned", [False, True])
def test_cfg0_tiny(kv, window_left, planned):
    w = workloads.cfg0_tiny(kv, device=DEV, quantize_fn=gpu_quantize, poison=True,
                            act_dtype=torch.bfloat16)  # fmt: skip
    before = _snapshot(w)
    out = run_decode(w, window_left=window_left, planned=planned)
    assert out.shape == w.q.shape and out.dtype == w.q.dtype
    _check_append(w, before)
    assert_close(out, expected_decode(w, window_left=window_left), *tolerances(kv), what=f"cfg0 {kv} w={window_left}")


@pytest.mark.parametrize("kv", ["bf16", "int8", "fp8"])
def test_split_invariance_and_determinism(kv):
    w = workloads.cfg0_tiny(kv, device=DEV, quantize_fn=gpu_quantize)
    outs = [run_decode(w, num_splits=n).float() for n in (1, 2, 8, 64)]
    for o in outs[1:]:
        assert (o - outs[0]).abs().max().item() < 2e-3  # same math, different partial boundaries
    again = run_decode(w, num_splits=8).float()
    assert torch.equal(again, outs[2]), "two identical calls must give identical bits"


def test_fp16_query_with_quantized_cache():
    w = workloads.cfg0_tiny("int8", device=DEV, quantize_fn=gpu_quantize, act_dtype=torch.float16)
    out = run_decode(w)
    assert out.dtype == torch.float16
    assert_close(out, expected_decode(w), *tolerances("int8"), what="fp16 q / int8 kv")


@pytest.mark.parametrize("kv,hq,hkv,d,bs", [
    ("bf16", 28, 4, 128, 16), ("int8", 28, 4, 128, 16), ("fp8", 32, 8, 128, 16), ("bf16", 16, 2, 128, 256),
    ("int8", 4, 4, 64, 16), ("bf16", 6, 2, 128, 16), ("fp16", 12, 1, 64, 32), ("int8", 5, 1, 128, 8),
    ("bf16", 8, 2, 96, 16), ("bf16", 24, 2, 128, 16), ("fp8", 8, 8, 128, 48), ("fp32", 8, 2, 128, 16),
    # more than 16 q heads per kv head: several 16-column tiles per kv head (2 x 16, 16 + 4, 16 + 16 + 8, 8 x 16)
    ("int8", 32, 1, 128, 16), ("bf16", 40, 2, 64, 16), ("fp8", 40, 1, 128, 16), ("bf16", 128, 1, 128, 16),
    ("int8", 136, 1, 64, 16),  # more than 128: the vector-ALU kernels
    ("bf16", 24, 4, 128, 12), ("int8", 8, 2, 128, 768),  # page sizes that are no power of two
    ("bf16", 4, 2, 64, 2),  # pages of fewer than 4 tokens: the vector-ALU kernels
])  # fmt: skip
def test_shapes_head_ratios_and_block_sizes(kv, hq, hkv, d, bs):
    g = torch.Generator().manual_seed(hq * 131 + d)
    batch = 6
    lengths = torch.randint(0, 700, (batch,), generator=g)
    lengths[0] = 0
    lengths[1] = bs - 1  # the append opens... the last slot of a page
    lengths[2] = bs  # ...and the first slot of a fresh page
    w = workloads.make_decode_workload("shapes", seed=77, batch=batch, hq=hq, hkv=hkv, d=d, bs=bs, kv=kv,
                                       lengths=lengths, device=DEV, quantize_fn=gpu_quantize, poison=True)  # fmt: skip
    before = _snapshot(w)
    out = run_decode(w)
    assert_close(out, expected_decode(w), *tolerances(kv), what=f"{kv} {hq}/{hkv} d={d} bs={bs}")
    _check_append(w, before)
    if kv != "fp32":  # through a plan: the same bits (the second append rewrites the slot with the same values)
        assert torch.equal(run_decode(w, planned=True), out)


@pytest.mark.parametrize("kv", ["bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("d", [256, 192, 512])
@pytest.mark.parametrize("hq,hkv,window_left", [(16, 8, None), (8, 2, None), (4, 1, 300), (24, 4, None), (40, 2, None)])
def test_head_dims_192_256_512_on_the_matrix_core_kernel(kv, d, hq, hkv, window_left):
    """Head dims 256 (Gemma-family sliding layers, Qwen3.5), 192 (128 + 64 rotary channels of MLA-style layers) and
    512 (Gemma-family full-attention layers): two, three resp. four waves share a head, each with a part of the head dimension, and exchange their parts of the
    scores.  Long and short rows so that units cross sequence borders, one kv head per workgroup so that the heads of
    a workgroup run different units, the append checked bit for bit."""
    g = torch.Generator().manual_seed(hq * 7 + hkv)
    batch = 9
    lengths = torch.randint(0, 2500, (batch,), generator=g)
    lengths[0], lengths[1], lengths[2] = 0, 15, 16
    w = workloads.make_decode_workload("wide", seed=79, batch=batch, hq=hq, hkv=hkv, d=d, bs=16, kv=kv,
                                       lengths=lengths, device=DEV, quantize_fn=gpu_quantize, poison=True)  # fmt: skip
    before = _snapshot(w)
    out = run_decode(w, window_left=window_left)
    assert_close(out, expected_decode(w, window_left=window_left), *tolerances(kv), what=f"D={d} {kv} {hq}/{hkv}")
    _check_append(w, before)
    # the same step through a plan: the same bits (the second append rewrites the slot with the same values)
    assert torch.equal(run_decode(w, window_left=window_left, planned=True), out)


def test_graph_padded_rows_on_a_scratch_block_are_harmless():
    """Rows with cache_seqlens = 0 and an all-scratch block table (how the decode graph pads a bucket)."""
    w = workloads.cfg0_tiny("bf16", device=DEV)
    nb = w.k_cache.shape[0]
    scratch = nb - 1
    assert not (w.block_table[:, :] == scratch)[:, :1].any()
    pad = 3
    w.q = torch.cat([w.q, torch.randn_like(w.q[:pad])])
    w.k_update = torch.cat([w.k_update, torch.randn_like(w.k_update[:pad])])
    w.v_update = torch.cat([w.v_update, torch.randn_like(w.v_update[:pad])])
    w.block_table = torch.cat([w.block_table, torch.full_like(w.block_table[:pad], scratch)])
    w.cache_seqlens = torch.cat([w.cache_seqlens, torch.zeros_like(w.cache_seqlens[:pad])])
    out = run_decode(w)
    assert torch.isfinite(out.float()).all()
    assert_close(out[:4], expected_decode(w, rows=slice(0, 4)), *tolerances("bf16"), what="live rows")


@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_cfg1_cfg2_full_size(kv):
    """Qwen2.5-7B-like shape at full size: B=64, 28/4 heads, D=128, ctx 512..4096."""
    w = workloads.cfg1_qwen7b(kv, device=DEV, quantize_fn=gpu_quantize, seed=1002 if kv == "int8" else 1001)
    before = _snapshot(w)
    out = run_decode(w)
    _check_append(w, before)
    assert torch.equal(run_decode(w, planned=True), out), "the planned step differs from the plain one"
    mx, mean = assert_close(out, expected_decode(w), *tolerances(kv), what=f"cfg {kv} full")
    print(f"cfg1/2 {kv}: max-abs {mx:.3e} mean-abs {mean:.3e}")
    # size-independent property: appending the same token again at L_b + 1 ... is a different op; instead
    # check linearity in V: doubling every V (update included) doubles the output
    if kv == "bf16":
        w2 = workloads.cfg1_qwen7b(kv, device=DEV, seed=1001)
        w2.v_cache *= 2
        w2.v_update = w2.v_update * 2
        out2 = run_decode(w2)
        assert torch.equal(out2.float(), out.float() * 2)


def test_cfg3_rollout_shared_prefix_reduced_and_tail():
    """32x8 rollout shape is large; parity on a reduced draw (same generator, fewer prompts, long tail kept)."""
    w = workloads.cfg3_rollout("fp8", device=DEV, quantize_fn=gpu_quantize, prompts=4, samples=8, cap=20000)
    before = _snapshot(w)
    out = run_decode(w)
    _check_append(w, before)
    assert_close(out, expected_decode(w), *tolerances("fp8"), what="cfg3 reduced")
    # rows of one prompt share prefix pages: block ids equal on the shared columns
    assert torch.equal(w.block_table[0, :8], w.block_table[7, :8])


def test_error_behaviour_matches_the_reference_shim():
    w = workloads.cfg0_tiny("bf16", device=DEV)
    args = [w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table, w.cache_seqlens]
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        ops.areno_paged_causal_attention_decode(w.q.cpu(), *args[1:])
    with pytest.raises(ValueError, match="expects q shaped"):
        ops.areno_paged_causal_attention_decode(w.q[0], *args[1:])
    with pytest.raises(ValueError, match="int32 block_table"):
        ops.areno_paged_causal_attention_decode(*args[:5], w.block_table.long(), w.cache_seqlens)
    with pytest.raises(RuntimeError, match="areno_paged_causal_attention_decode.*dtype mismatch"):
        ops.areno_paged_causal_attention_decode(w.q.half(), *args[1:])
    with pytest.raises(RuntimeError, match="q heads must be divisible"):
        ops.areno_paged_causal_attention_decode(w.q[:, :7].contiguous(), *args[1:])
    with pytest.raises(RuntimeError, match="num_splits must be >= 1"):
        ops.areno_paged_causal_attention_decode(*args, num_splits=0)
    empty = ops.areno_paged_causal_attention_decode(w.q[:0], w.k_update[:0], w.v_update[:0], w.k_cache, w.v_cache,
                                                    w.block_table[:0], w.cache_seqlens[:0])  # fmt: skip
    assert empty.shape == (0, 8, 64)
    # as in the reference the op records a backward when an input asks for one (tests/test_gpu_backward.py), and none
    # under no_grad
    q_grad = w.q.clone().requires_grad_(True)
    assert ops.areno_paged_causal_attention_decode(q_grad, *args[1:]).requires_grad
    with torch.no_grad():
        assert not ops.areno_paged_causal_attention_decode(q_grad, *args[1:]).requires_grad
    # update rows that require grad keep the output in the graph; their gradient is None, as in the reference
    ku = w.k_update.clone().requires_grad_(True)
    out = ops.areno_paged_causal_attention_decode(w.q, ku, *args[2:])
    assert out.requires_grad
    out.float().sum().backward()
    assert ku.grad is None


def test_float64_tensors_compute_in_fp32_like_the_reference():
    """The reference's launchers take double tensors and accumulate in float (attention.cu:846,979 there)."""
    w = workloads.cfg0_tiny("fp32", device=DEV, poison=True, act_dtype=torch.float32)
    q, ku, vu = w.q.double(), w.k_update.double() + 1e-12, w.v_update.double() - 1e-12
    kc, vc = w.k_cache.double(), w.v_cache.double()
    out = ops.areno_paged_causal_attention_decode(q, ku, vu, kc, vc, w.block_table, w.cache_seqlens,
                                                  softmax_scale=w.softmax_scale)  # fmt: skip
    assert out.dtype == torch.float64
    ids, offs = qr.decode_addresses(w.block_table.cpu(), w.cache_seqlens.cpu(), w.k_cache.shape[1])
    assert torch.equal(kc.cpu()[ids, offs], ku.cpu()) and torch.equal(vc.cpu()[ids, offs], vu.cpu())  # the doubles as they are
    w.k_cache, w.v_cache = kc.float(), vc.float()
    assert_close(out, expected_decode(w), 1e-4, what="float64 decode")
    # varlen and dense ops
    g = torch.Generator(device=DEV).manual_seed(3)
    qv = torch.randn(40, 4, 64, generator=g, device=DEV, dtype=torch.float64)
    kv = torch.randn(40, 2, 64, generator=g, device=DEV, dtype=torch.float64)
    vv = torch.randn(40, 2, 64, generator=g, device=DEV, dtype=torch.float64)
    cu = torch.tensor([0, 7, 40], dtype=torch.int32, device=DEV)
    got = ops.areno_varlen_causal_attention(qv, kv, vv, cu)
    want = ops.areno_varlen_causal_attention(qv.float(), kv.float(), vv.float(), cu)
    assert got.dtype == torch.float64 and torch.equal(got.float(), want)
    qd = qv[:32].view(2, 16, 4, 64).transpose(1, 2).contiguous()
    kd = kv[:32].view(2, 16, 2, 64).transpose(1, 2).repeat_interleave(2, dim=1).contiguous()
    got = ops.areno_causal_attention(qd, kd, kd)
    assert got.dtype == torch.float64 and torch.equal(got.float(), ops.areno_causal_attention(qd.float(), kd.float(), kd.float()))


# ---- prefix groups: shared pages read once for several rows --------------------------------------------------------
def _grouped_decode(w, **kw):
    return ops.areno_paged_causal_attention_decode(
        w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table, w.cache_seqlens,
        softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale,
        prefix_group_rows=w.meta["prefix_group_rows"], shared_prefix_lens=w.meta["shared_prefix_lens"], **kw,
    )  # fmt: skip


@pytest.mark.parametrize("kv,hq,hkv,samples", [("fp8", 32, 8, 8), ("int8", 28, 4, 4), ("bf16", 8, 2, 3), ("fp8", 8, 8, 5)])
def test_prefix_groups_match_the_plain_op_and_the_oracle(kv, hq, hkv, samples):
    """Rollout batches at reduced size: 4 / 2 / 4 / 16 rows side by side, groups that do not fill the columns, prompts
    shorter than a tile (nothing to share) next to long ones."""
    w = workloads.cfg3_rollout(kv, device=DEV, prompts=6, samples=samples, prefix_lo=8, prefix_hi=700, median=120.0,
                               cap=900, quantize_fn=gpu_quantize, seed=77, hq=hq, hkv=hkv, poison=True)  # fmt: skip
    snapshot = tuple(None if t is None else t.clone() for t in (w.k_cache, w.v_cache, w.k_scale, w.v_scale))
    plain = run_decode(w)
    after_plain = tuple(None if t is None else t.clone() for t in (w.k_cache, w.v_cache, w.k_scale, w.v_scale))
    for dst, src in zip((w.k_cache, w.v_cache, w.k_scale, w.v_scale), snapshot):
        if dst is not None:
            dst.copy_(src)
    grouped = _grouped_decode(w)
    assert_close(grouped, expected_decode(w), *tolerances(kv), what=f"grouped {kv} vs oracle")
    assert torch.equal(_grouped_decode(w, plan=build_plan(w, grouped=True)), grouped), "planned grouped step differs"
    # same math in another summation order: the outputs may differ by one unit of the 16-bit output format
    assert_close(grouped, plain.cpu().float(), 8e-3, what=f"grouped {kv} vs plain op")
    for a, b, name in zip((w.k_cache, w.v_cache, w.k_scale, w.v_scale), after_plain, ("k", "v", "k_scale", "v_scale")):
        if a is not None:
            same = a.view(torch.uint8) == b.view(torch.uint8)
            assert bool(same.all()), f"{name}: the append differs between the grouped and the plain op"


def test_cfg3_full_size_grouped():
    """The rollout configuration at its stated size, through the prefix-group kernel the benchmark times: 32 prompts x 8
    samples, 32 / 8 heads, fp8 pages with fp32 scales, prefixes U[256, 2048], continuations lognormal capped at 32 768
    (block tables ~2 100 columns wide).  The append is checked bit for bit over the whole pool; the output against the
    oracle on one whole group, the eight longest rows, the shortest row and the last row, and against the plain op
    (every row reading its own pages) on all 256 rows."""
    w = workloads.cfg3_rollout("fp8", device=DEV, quantize_fn=gpu_quantize)
    assert w.q.shape == (256, 32, 128) and w.meta["prefix_group_rows"] == 8
    pools = (w.k_cache, w.v_cache, w.k_scale, w.v_scale)
    on_device = tuple(t.clone() for t in pools)
    before = _snapshot(w)
    grouped = _grouped_decode(w)
    torch.cuda.synchronize()
    _check_append(w, before)
    del before
    lens = w.cache_seqlens.cpu()
    order = torch.argsort(lens, descending=True)
    longest_group = int(order[0]) // 8
    rows = sorted(set(range(8 * longest_group, 8 * longest_group + 8)) | set(order[:8].tolist()) | {int(order[-1]), 255})
    print(f"cfg3 full: longest row {int(lens.max())} tokens, table {tuple(w.block_table.shape)}, oracle rows {rows}")
    want = expected_decode_rows(w, rows)
    mx, mean = assert_close(grouped[rows], want, *tolerances("fp8"), what="cfg3 full size, grouped kernel vs oracle")
    print(f"cfg3 full grouped: max-abs {mx:.3e} mean-abs {mean:.3e} on {len(rows)} rows")
    after_grouped = tuple(t.clone() for t in pools)
    assert torch.equal(_grouped_decode(w, plan=build_plan(w, grouped=True)), grouped), "planned grouped step differs"
    for dst, src in zip(pools, on_device):
        dst.copy_(src)
    plain = run_decode(w)
    assert_close(grouped, plain.cpu().float(), 8e-3, what="cfg3 full size, grouped vs plain op, all rows")
    for a, b, name in zip(pools, after_grouped, ("k", "v", "k_scale", "v_scale")):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{name}: grouped and plain appends differ"


def test_batches_beyond_one_launch_run_in_row_ranges():
    """More rows than the matrix-core kernel indexes in one launch (1024): the library runs row ranges one after the
    other; plain rows (1500) and rollout groups of 3 (1200 rows: ranges end on group borders)."""
    g = torch.Generator().manual_seed(5)
    lengths = torch.randint(0, 90, (1500,), generator=g)
    w = workloads.make_decode_workload("wide-batch", seed=81, batch=1500, hq=8, hkv=2, d=128, bs=16, kv="int8",
                                       lengths=lengths, device=DEV, quantize_fn=gpu_quantize, poison=True)  # fmt: skip
    before = _snapshot(w)
    out = run_decode(w)
    assert_close(out, expected_decode(w), *tolerances("int8"), what="1500 rows")
    _check_append(w, before)
    plan = build_plan(w)
    assert plan.units == 0  # a plan covers one launch; the op then runs as without one
    assert torch.equal(run_decode(w, planned=True), out)
    r = workloads.cfg3_rollout("fp8", device=DEV, prompts=400, samples=3, prefix_lo=40, prefix_hi=120, median=30.0,
                               cap=100, quantize_fn=gpu_quantize, seed=83, hq=8, hkv=2)  # fmt: skip
    grouped = _grouped_decode(r)
    assert_close(grouped, expected_decode(r), *tolerances("fp8"), what="1200 grouped rows")


def test_prefix_groups_clip_an_overstated_shared_length():
    """shared_prefix_lens larger than what a row has cached is clipped to the shortest row of the group."""
    w = workloads.cfg3_rollout("fp8", device=DEV, prompts=3, samples=4, prefix_lo=64, prefix_hi=200, median=50.0,
                               cap=300, quantize_fn=gpu_quantize, seed=78, hq=8, hkv=2)  # fmt: skip
    # claim far more than the prompts hold: only identical pages may be merged, so this must still be exact whenever
    # the claim is cut back to the rows' cached lengths (rows of a group differ only behind the prompt here)
    w.meta["shared_prefix_lens"] = w.meta["shared_prefix_lens"].clone()
    w.meta["shared_prefix_lens"][1] = 0  # and one group that shares nothing
    out = _grouped_decode(w)
    assert_close(out, expected_decode(w), *tolerances("fp8"), what="clipped shared length")


def test_prefix_groups_argument_checks():
    w = workloads.cfg3_rollout("fp8", device=DEV, prompts=2, samples=4, prefix_lo=64, prefix_hi=100, median=30.0, cap=100,
                               quantize_fn=gpu_quantize, seed=79, hq=8, hkv=2)  # fmt: skip
    with pytest.raises(ValueError, match="together"):
        ops.areno_paged_causal_attention_decode(w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table,
                                                w.cache_seqlens, k_scale=w.k_scale, v_scale=w.v_scale,
                                                prefix_group_rows=4)  # fmt: skip
    with pytest.raises(ValueError, match="multiple of prefix_group_rows"):
        ops.areno_paged_causal_attention_decode(w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table,
                                                w.cache_seqlens, k_scale=w.k_scale, v_scale=w.v_scale,
                                                prefix_group_rows=3, shared_prefix_lens=w.meta["shared_prefix_lens"])  # fmt: skip
    # a window switches the grouping off, the result is the plain op's
    out = _grouped_decode(w, window_left=40)
    assert_close(out, expected_decode(w, window_left=40), *tolerances("fp8"), what="window with groups")


@pytest.mark.parametrize("seed", range(48))
def test_random_draws_of_shape_length_window_and_cache_type(seed):
    """Seeded random configurations through the whole op: cache type, head counts, head dim, page size, batch, window and
    length distribution (empty rows, rows of a few tokens next to long ones, many short rows so that a wave's share of
    the tiles crosses several rows).  Output against the oracle, append bit for bit over the whole pool."""
    import random

    rng = random.Random(1000 + seed)
    kv = rng.choice(["bf16", "fp16", "int8", "fp8"])
    hkv = rng.choice([1, 2, 4, 8])
    group = rng.choice([1, 2, 4, 7, 8, 16, 20, 33])  # above 16: several column tiles per kv head
    d = rng.choice([64, 128])
    bs = rng.choice([4, 8, 12, 16, 32, 48, 64])  # 12, 48: the page arithmetic's division by multiply and shift
    batch = rng.choice([1, 3, 17, 64, 130])
    profile = rng.choice(["short", "mixed", "long"])
    g = torch.Generator().manual_seed(seed)
    if profile == "short":
        lengths = torch.randint(0, 40, (batch,), generator=g)
    elif profile == "mixed":
        lengths = torch.where(torch.rand(batch, generator=g) < 0.7, torch.randint(0, 60, (batch,), generator=g),
                              torch.randint(200, 3000, (batch,), generator=g))  # fmt: skip
    else:
        lengths = torch.randint(500, 2500, (batch,), generator=g)
    window = rng.choice([None, None, 0, 33, 700])
    w = workloads.make_decode_workload(f"draw-{seed}", seed=500 + seed, batch=batch, hq=hkv * group, hkv=hkv, d=d, bs=bs,
                                       kv=kv, lengths=lengths, device=DEV, quantize_fn=gpu_quantize, poison=True,
                                       act_dtype=torch.float16 if kv == "fp16" else torch.bfloat16)  # fmt: skip
    before = _snapshot(w)
    out = run_decode(w, window_left=window)
    what = f"draw {seed}: {kv} {hkv * group}/{hkv} d={d} bs={bs} batch={batch} {profile} window={window}"
    assert_close(out, expected_decode(w, window_left=window), *tolerances(kv), what=what)
    _check_append(w, before)
    assert torch.equal(run_decode(w, window_left=window, planned=True), out), f"{what}: the planned step differs"


def test_a_plan_for_other_shapes_is_refused():
    w = workloads.cfg0_tiny("int8", device=DEV, quantize_fn=gpu_quantize)
    plan = build_plan(w)
    assert plan.units > 0 and plan.batch == w.q.shape[0]
    args = (w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table, w.cache_seqlens)
    kw = dict(softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale, plan=plan)
    with pytest.raises(RuntimeError, match="plan was built for other shapes"):
        ops.areno_paged_causal_attention_decode(*args, window_left=5, **kw)
    with pytest.raises(RuntimeError, match="plan was built for other shapes"):
        ops.areno_paged_causal_attention_decode(w.q[:3], w.k_update[:3], w.v_update[:3], w.k_cache, w.v_cache,
                                                w.block_table[:3].contiguous(), w.cache_seqlens[:3], **kw)  # fmt: skip
    with pytest.raises(ValueError, match="int32 block_table"):
        ops.areno_paged_decode_plan(w.block_table.long(), w.cache_seqlens, w.k_cache, w.v_cache, q_heads=8,
                                    k_scale=w.k_scale, v_scale=w.v_scale)  # fmt: skip


def test_one_plan_serves_the_layers_of_a_step():
    """Two layers (two cache pools) of one decode step share block table, lengths and one plan."""
    layers = [workloads.cfg0_tiny("fp8", device=DEV, quantize_fn=gpu_quantize, seed=s) for s in (1000, 1000)]
    a, b = layers
    b.k_cache.copy_(torch.flip(a.k_cache.view(torch.uint8), dims=(3,)).view(b.k_cache.dtype))  # other contents, same tables
    plan = build_plan(a)
    for w in layers:
        plain = run_decode(w)
        with_plan = ops.areno_paged_causal_attention_decode(
            w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, a.block_table, a.cache_seqlens,
            softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale, plan=plan)  # fmt: skip
        assert torch.equal(with_plan, plain)
        assert_close(with_plan, expected_decode(w), *tolerances("fp8"), what="layer through the shared plan")


@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_a_row_at_the_end_of_its_block_table_writes_nothing(kv):
    """A row whose length equals the table's capacity (no column for the next position: the page bookkeeping reports
    it as full) must not have its new token stored anywhere -- the cache writer skips such rows -- and no kernel may
    read a column behind the table; the other rows decode as usual."""
    bs, cols = 16, 6
    lengths = torch.tensor([cols * bs, 40, cols * bs, 7])
    w = workloads.make_decode_workload("full-rows", seed=91, batch=4, hq=8, hkv=2, d=128, bs=bs, kv=kv, lengths=lengths,
                                       device=DEV, quantize_fn=gpu_quantize, poison=True)  # fmt: skip
    w.block_table = w.block_table[:, :cols].contiguous()  # rows 0 and 2 fill their six columns
    before = _snapshot(w)
    for planned in (False, True):
        out = run_decode(w, planned=planned)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        live = [1, 3]
        ids, offs = qr.decode_addresses(w.block_table[live].cpu(), w.cache_seqlens[live].cpu(), bs)
        touched = torch.zeros(w.k_cache.shape[:2], dtype=torch.bool)
        touched[ids, offs] = True
        for name, old in zip(("k_cache", "v_cache", "k_scale", "v_scale"), before):
            if old is None:
                continue
            new = getattr(w, name).cpu()
            same = new.view(torch.uint8)[~touched] == old.view(torch.uint8)[~touched]
            assert same.all(), f"{name}: a slot other than the two served rows' targets changed"
        assert_close(out[live], expected_decode(w, rows=live), *tolerances(kv), what=f"served rows, planned={planned}")
