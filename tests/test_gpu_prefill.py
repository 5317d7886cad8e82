"""Varlen prefill ops vs the CPU oracle: packed new-token attention (the reference's op) and
causal prefill over paged, optionally quantized KV with a cached context (this build's extension)."""

import pytest
import torch

from areno_amd import workloads
from areno_amd.accel import attention as ops
from oracle import attention_ref as ar
from tests.gpu_util import DEV, assert_close, compact_pages, dequant_cpu, gpu_quantize, tolerances

pytestmark = pytest.mark.gpu


def _packed(lens, hq, hkv, d, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    t = sum(lens)
    q, k, v = (torch.randn(t, h, d, generator=g).to(dtype) for h in (hq, hkv, hkv))
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    return q, k, v, cu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("window_left", [None, 0, 7])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (28, 4, 128), (4, 4, 80), (8, 2, 256), (6, 6, 192), (8, 2, 512), (40, 2, 128)])
def test_varlen_new_tokens_only(dtype, window_left, hq, hkv, d):
    q, k, v, cu = _packed([5, 1, 130, 0, 67], hq, hkv, d, dtype)
    out = ops.areno_varlen_causal_attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), window_left=window_left)
    want = ar.ref_varlen(q, k, v, cu, ar.window_left_arg(window_left), d**-0.5)
    assert out.dtype == dtype and out.shape == q.shape
    assert_close(out, want, *tolerances("bf16"), what="varlen")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128, 192, 256, 512])
@pytest.mark.parametrize("profile", ["climb", "jump", "fall", "wide"])
def test_varlen_score_ranges_that_move_along_the_keys(dtype, d, profile):
    """The matrix-core kernel keeps a softmax reference value per row that it raises only when a key tile exceeds it
    by a margin, so rows whose scores climb slowly (the reference lags), jump far (a late raise rescales everything
    before it), fall (the first tile dominates) or spread over a wide range all have to come out like the oracle's
    exact-maximum softmax."""
    lens = [300, 33, 1, 150]
    q, k, v, cu = _packed(lens, 4, 2, d, torch.float32, seed=d)
    pos = torch.cat([torch.arange(n, dtype=torch.float32) for n in lens])
    if profile == "climb":  # a shared direction whose weight grows by a little per key
        gain = 0.02 * pos
    elif profile == "jump":  # every 97th key scores far above its neighbours
        gain = torch.where(pos % 97 == 96, 9.0, 0.0)
    elif profile == "fall":
        gain = 6.0 - 0.03 * pos
    else:
        gain = torch.zeros_like(pos)
        q, k = 5.0 * q, 5.0 * k
    direction = torch.ones(d) * (d**-0.5)
    q = q + 2.0 * (d**0.25) * direction  # every query has a component along the shared direction
    k = k + gain[:, None, None] * (d**0.25) * direction
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    out = ops.areno_varlen_causal_attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV))
    want = ar.ref_varlen(q, k, v, cu, ar.window_left_arg(None), d**-0.5)
    assert_close(out, want, *tolerances("bf16"), what=f"varlen {profile}")


def _expected_prefill(w, window_left=None):
    kc, vc = dequant_cpu(w.k_cache, w.k_scale), dequant_cpu(w.v_cache, w.v_scale)
    return ar.ref_paged_varlen_prefill(w.q.cpu().float(), kc, vc, w.block_table.cpu(), w.cu_seqlens_q.cpu(),
                                       w.context_lens.cpu(), ar.window_left_arg(window_left), w.softmax_scale)  # fmt: skip


def _run_prefill(w, window_left=None):
    return ops.areno_paged_varlen_causal_attention(
        w.q, w.k_cache, w.v_cache, w.block_table, w.cu_seqlens_q, w.context_lens,
        window_left=window_left, softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale,
    )  # fmt: skip


@pytest.mark.parametrize("kv", ["bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("window_left", [None, 33])
def test_paged_prefill_small(kv, window_left):
    w = workloads.cfg4_prefill(kv, device=DEV, seqs=5, new_hi=70, ctx_hi=300, quantize_fn=gpu_quantize, seed=5)
    out = _run_prefill(w, window_left)
    assert_close(out, _expected_prefill(w, window_left), *tolerances(kv), what=f"paged prefill {kv}")


@pytest.mark.parametrize("hq,hkv,d,bs", [
    (28, 4, 128, 16), (8, 8, 64, 32), (6, 2, 128, 256), (4, 1, 96, 16),
    # more than 16 q heads per kv head: several workgroup rows per kv head, 16 q heads each (16 + 16, 16 + 4, 16 + 8 at
    # head dim 256, 16 + 16 + 1)
    (32, 1, 128, 16), (40, 2, 64, 32), (24, 1, 256, 16), (33, 1, 128, 16),
    # page sizes that are no power of two: the key's page by a multiplication and a shift
    (28, 4, 128, 12), (8, 2, 64, 48), (16, 8, 512, 80), (8, 8, 128, 1000),
])  # fmt: skip
def test_paged_prefill_shapes(hq, hkv, d, bs):
    g = torch.Generator().manual_seed(d + hq)
    new = torch.tensor([1, 64, 17, 129])
    ctx = torch.tensor([0, 5, 200, 63])
    w = workloads.make_prefill_workload("shapes", seed=3, new_lens=new, ctx_lens=ctx, hq=hq, hkv=hkv, d=d, bs=bs,
                                        kv="bf16", device=DEV)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances("bf16"), what="prefill shapes")


@pytest.mark.parametrize("kv", ["bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("d", [256, 192, 512])
@pytest.mark.parametrize("hq,hkv,window_left", [(16, 8, None), (8, 1, 40), (12, 4, None)])
def test_paged_prefill_head_dims_192_256_512(kv, d, hq, hkv, window_left):
    """Head dims 256 (the sliding-attention layers of the Gemma family, Qwen3.5), 192 (128 + 64 rotary channels of
    the MLA-style layers) and 512 (the Gemma family's full-attention layers) on the matrix-core kernel: one 16-row
    tile per wave, at 512 shared by two waves with half of the head each; a query block cut by many shares goes
    through the merge of the wide partials."""
    new = torch.tensor([3, 150, 64, 1, 33])
    ctx = torch.tensor([900, 0, 77, 2500, 310])
    w = workloads.make_prefill_workload("wide", seed=11 + hq, new_lens=new, ctx_lens=ctx, hq=hq, hkv=hkv, d=d, bs=16,
                                        kv=kv, device=DEV, quantize_fn=gpu_quantize)  # fmt: skip
    assert_close(_run_prefill(w, window_left), _expected_prefill(w, window_left), *tolerances(kv),
                 what=f"prefill D={d} {kv}")  # fmt: skip


@pytest.mark.parametrize("kv", ["bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("d,bs", [(64, 16), (64, 64), (128, 8), (128, 128), (64, 24), (128, 5), (128, 100)])
def test_paged_prefill_staging_schemes(kv, d, bs):
    """The staging of a key tile has two schemes: one K and one V chunk per thread and round, or, when a tile has at
    most one chunk per thread (8-bit tiles up to head dim 128, 16-bit tiles at 64), K staged by the first half of
    the workgroup and V by the second.  8-bit tiles at head dim 64 leave half of each half without a live chunk.
    Page sizes below, at and above the 32-key tile, powers of two and others."""
    new = torch.tensor([70, 1, 200, 33])
    ctx = torch.tensor([0, 1300, 95, 640])
    w = workloads.make_prefill_workload("staging", seed=d + bs, new_lens=new, ctx_lens=ctx, hq=8, hkv=2, d=d, bs=bs,
                                        kv=kv, device=DEV, quantize_fn=gpu_quantize)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances(kv), what=f"prefill staging D={d} {kv} page {bs}")


@pytest.mark.parametrize("seed", range(32))
def test_random_draws_of_prefill_shape_length_window_and_cache_type(seed):
    """Seeded random configurations through the paged prefill op: cache type, head counts (up to 33 q heads per kv
    head: several workgroup rows per kv head), head dim (one tile or two per wave, the head split over two waves at
    512, 96 on the one-wave-per-row kernel), page size (12 and 48: no power of two), number of sequences, new and
    cached lengths (sequences without new tokens, single tokens, blocks cut by many shares) and window."""
    import random

    rng = random.Random(7000 + seed)
    kv = rng.choice(["bf16", "fp16", "int8", "fp8"])
    group = rng.choice([1, 2, 4, 7, 8, 16, 20, 33])
    hkv = rng.choice([h for h in (1, 2, 4, 8) if h * group <= 64])
    d = rng.choice([64, 128, 128, 192, 256, 512, 96])
    bs = rng.choice([8, 16, 32, 64, 256, 12, 48])
    slow = d == 96  # one wave per (token, head): keep the work small
    seqs = rng.choice([1, 3, 9] if slow else [1, 3, 9, 40])
    g = torch.Generator().manual_seed(seed)
    new_profile = rng.choice(["ones", "short", "mixed", "long"])
    if new_profile == "ones":
        new = torch.randint(0, 2, (seqs,), generator=g)
    elif new_profile == "short":
        new = torch.randint(0, 20, (seqs,), generator=g)
    elif new_profile == "mixed":
        new = torch.where(torch.rand(seqs, generator=g) < 0.6, torch.randint(0, 9, (seqs,), generator=g),
                          torch.randint(60, 300, (seqs,), generator=g))  # fmt: skip
    else:
        new = torch.randint(100, 140 if slow else 400, (seqs,), generator=g)
    if int(new.sum()) == 0:
        new[0] = 1
    ctx_hi = 300 if slow else rng.choice([1, 90, 700, 4000])
    ctx = torch.where(torch.rand(seqs, generator=g) < 0.3, torch.zeros(seqs, dtype=torch.int64),
                      torch.randint(0, ctx_hi, (seqs,), generator=g))  # fmt: skip
    window = rng.choice([None, None, 0, 33, 700])
    w = workloads.make_prefill_workload(f"draw-{seed}", seed=900 + seed, new_lens=new, ctx_lens=ctx, hq=hkv * group,
                                        hkv=hkv, d=d, bs=bs, kv=kv, device=DEV, quantize_fn=gpu_quantize,
                                        act_dtype=torch.float16 if kv == "fp16" else torch.bfloat16)  # fmt: skip
    what = f"draw {seed}: {kv} {hkv * group}/{hkv} d={d} bs={bs} seqs={seqs} new={new_profile} ctx<{ctx_hi} window={window}"
    assert_close(_run_prefill(w, window), _expected_prefill(w, window), *tolerances(kv), what=what)


def test_prefill_with_a_full_sequence_list():
    """1024 sequences, the most one launch of the matrix-core kernel indexes: the prefix sum over the sequences must
    also produce its last entry, the total."""
    g = torch.Generator().manual_seed(3)
    new = torch.randint(1, 4, (1024,), generator=g)
    ctx = torch.randint(0, 40, (1024,), generator=g)
    w = workloads.make_prefill_workload("full-list", seed=31, new_lens=new, ctx_lens=ctx, hq=4, hkv=2, d=64, bs=16,
                                        kv="bf16", device=DEV)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances("bf16"), what="1024 sequences")


def test_write_then_prefill_then_decode_are_consistent():
    """The three ops agree with each other: cache write of the new tokens, prefill with ctx,
    and n = 1 prefill == decode without append."""
    w = workloads.cfg4_prefill("fp8", device=DEV, seqs=6, new_hi=40, ctx_hi=200, quantize_fn=gpu_quantize, seed=9)
    ops.areno_paged_cache_write(w.k_new, w.v_new, w.k_cache, w.v_cache, w.cache_block_ids, w.cache_block_offsets,
                                k_scale=w.k_scale, v_scale=w.v_scale)  # fmt: skip
    out = _run_prefill(w)
    assert_close(out, _expected_prefill(w), *tolerances("fp8"), what="after write")
    # last query of each sequence == a decode row whose token is already cached: compare through the oracle
    cu = w.cu_seqlens_q.cpu().long()
    last = cu[1:] - 1
    lens = (w.context_lens.cpu().long() + (cu[1:] - cu[:-1]) - 1).int()
    kc, vc = dequant_cpu(w.k_cache, w.k_scale), dequant_cpu(w.v_cache, w.v_scale)
    dec = ar.ref_paged_decode(w.q.cpu().float()[last], kc, vc, w.block_table.cpu(), lens, -1, w.softmax_scale)
    assert_close(out[last.to(DEV)], dec, *tolerances("fp8"), what="prefill last row vs decode oracle")


def test_cfg4_reduced():
    """cfg 4 shape (32/8 heads, D=128, fp8) with the full range of new lengths and a reduced context range."""
    w = workloads.cfg4_prefill("fp8", device=DEV, seqs=6, new_hi=512, ctx_hi=3000, quantize_fn=gpu_quantize)
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances("fp8"), what="cfg4 reduced")


def test_cfg4_full_size():
    """cfg 4 at its stated size: 16 sequences, 1..512 new tokens on 0..16 384 cached ones, 32 / 8 heads, fp8 pages.  The new
    tokens go through the quantizing cache write first, as in the op sequence the benchmark times.  Every sequence is checked
    against the oracle on its first and last query row and 16 random ones in between (a row sees all of its sequence's keys
    up to its own position, so the long contexts are covered by every sampled row)."""
    w = workloads.cfg4_prefill("fp8", device=DEV, quantize_fn=gpu_quantize)
    assert w.context_lens.shape == (16,)
    ops.areno_paged_cache_write(w.k_new, w.v_new, w.k_cache, w.v_cache, w.cache_block_ids, w.cache_block_offsets,
                                k_scale=w.k_scale, v_scale=w.v_scale)  # fmt: skip
    out = _run_prefill(w)
    torch.cuda.synchronize()
    got = out.cpu().float()
    assert torch.isfinite(got).all()
    cu = w.cu_seqlens_q.cpu().tolist()
    ctx = w.context_lens.cpu().tolist()
    print(f"cfg4 full: new {[cu[i + 1] - cu[i] for i in range(16)]} ctx {ctx}")
    g = torch.Generator().manual_seed(4)
    hq, hkv = w.q.shape[1], w.k_cache.shape[2]
    worst = 0.0
    for s in range(16):
        n = cu[s + 1] - cu[s]
        picks = sorted({0, n - 1} | set(torch.randint(0, n, (16,), generator=g).tolist()))
        bs = w.k_cache.shape[1]
        cols = (ctx[s] + n + bs - 1) // bs
        table = w.block_table[s : s + 1, :cols].cpu()
        kc, compact = compact_pages(w.k_cache, w.k_scale, table)
        vc, _ = compact_pages(w.v_cache, w.v_scale, table)
        k = ar.gather_paged(kc, compact[0], ctx[s] + n).repeat_interleave(hq // hkv, dim=1).transpose(0, 1).unsqueeze(0)
        v = ar.gather_paged(vc, compact[0], ctx[s] + n).repeat_interleave(hq // hkv, dim=1).transpose(0, 1).unsqueeze(0)
        for i in picks:
            upto = ctx[s] + i + 1
            q1 = w.q[cu[s] + i].cpu().float().view(1, hq, 1, -1)
            want = ar.ref_attention(q1, k[:, :, :upto], v[:, :, :upto], ctx[s] + i, -1, w.softmax_scale).view(hq, -1)
            err = (got[cu[s] + i] - want).abs().max().item()
            worst = max(worst, err)
            assert err <= tolerances("fp8")[0], f"cfg4 full: sequence {s} (ctx {ctx[s]}, new {n}) row {i}: max-abs {err:.4g}"
    print(f"cfg4 full: max-abs {worst:.3e} over the sampled rows")


@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_prefill_one_query_block_cut_by_many_shares(kv):
    """A single short chunk on a long context: every workgroup owns a slice of the same query block's keys, so the
    result only exists after the merge of all their partials."""
    w = workloads.make_prefill_workload("long-ctx", seed=21, new_lens=torch.tensor([9]), ctx_lens=torch.tensor([6000]),
                                        hq=8, hkv=2, d=128, bs=16, kv=kv, device=DEV, quantize_fn=gpu_quantize)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances(kv), what="one block, many shares")


def test_prefill_sequences_without_new_tokens_and_single_tokens():
    """Empty chunks (cu_seqlens repeats) between chunks of 1, 33 and 200 tokens; contexts 0, tile-aligned and odd."""
    new = torch.tensor([0, 1, 0, 33, 1, 0, 200, 0])
    ctx = torch.tensor([50, 0, 0, 64, 1023, 7, 31, 0])
    w = workloads.make_prefill_workload("ragged", seed=22, new_lens=new, ctx_lens=ctx, hq=12, hkv=4, d=64, bs=32,
                                        kv="fp8", device=DEV, quantize_fn=gpu_quantize)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances("fp8"), what="ragged chunks")


@pytest.mark.parametrize("window_left", [0, 31, 32, 100, 5000])
def test_prefill_window_moves_the_first_tile(window_left):
    """Sliding windows shorter than, equal to and longer than a key tile, and longer than every context."""
    new = torch.tensor([70, 3, 130])
    ctx = torch.tensor([900, 40, 0])
    w = workloads.make_prefill_workload("window", seed=23, new_lens=new, ctx_lens=ctx, hq=8, hkv=2, d=128, bs=16,
                                        kv="bf16", device=DEV)  # fmt: skip
    assert_close(_run_prefill(w, window_left), _expected_prefill(w, window_left), *tolerances("bf16"),
                 what=f"window {window_left}")  # fmt: skip


def test_prefill_many_sequences():
    """More sequences than workgroup shares per kv head: most shares hold several whole query blocks."""
    g = torch.Generator().manual_seed(24)
    new = torch.randint(1, 40, (300,), generator=g)
    ctx = torch.randint(0, 90, (300,), generator=g)
    w = workloads.make_prefill_workload("many", seed=24, new_lens=new, ctx_lens=ctx, hq=8, hkv=8, d=64, bs=16,
                                        kv="int8", device=DEV, quantize_fn=gpu_quantize)  # fmt: skip
    assert_close(_run_prefill(w), _expected_prefill(w), *tolerances("int8"), what="many sequences")


def test_prefill_c_abi_rejects_a_short_workspace():
    from areno_amd.accel import cabi

    w = workloads.cfg4_prefill("fp8", device=DEV, seqs=2, new_hi=8, ctx_hi=40, quantize_fn=gpu_quantize, seed=5)
    cache = cabi.describe_cache(w.k_cache, w.v_cache, w.k_scale, w.v_scale)
    need = cabi.prefill_workspace_bytes(w.k_cache.shape[2], w.k_cache.shape[3])
    assert need > 0
    out = torch.empty_like(w.q)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)

    def call(nbytes):
        return cabi.paged_varlen_prefill(cache, w.q, out, w.block_table, w.cu_seqlens_q, w.context_lens, ws,
                                         softmax_scale=w.softmax_scale, workspace_bytes=nbytes)  # fmt: skip

    assert call(need - 1) == cabi.ERR_WORKSPACE
    assert b"workspace" in cabi.lib().areno_hip_last_error()
    assert call(need) == 0
    torch.cuda.synchronize()
    assert_close(out, _expected_prefill(w), *tolerances("fp8"), what="c abi prefill")


def test_dense_causal_attention_wrapper():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(2, 4, 9, 64, generator=g).bfloat16()
    k = torch.randn(2, 4, 21, 64, generator=g).bfloat16()
    v = torch.randn(2, 4, 21, 64, generator=g).bfloat16()
    out = ops.areno_causal_attention(q.to(DEV), k.to(DEV), v.to(DEV), query_start=12, window_left=6)
    want = ar.ref_attention(q, k, v, 12, 6, 64**-0.5)
    assert_close(out, want, *tolerances("bf16"), what="dense")


def test_varlen_error_behaviour():
    q, k, v, cu = _packed([4, 4], 4, 2, 64, torch.bfloat16)
    with pytest.raises(RuntimeError, match="requires CUDA"):
        ops.areno_varlen_causal_attention(q, k, v, cu)
    q, k, v, cu = (t.to(DEV) for t in (q, k, v, cu))
    with pytest.raises(ValueError, match="int32 1D cu_seqlens"):
        ops.areno_varlen_causal_attention(q, k, v, cu.long())
    with pytest.raises(ValueError, match="token count mismatch"):
        ops.areno_varlen_causal_attention(q, k[:-1], v, cu)
    with pytest.raises(ValueError, match="divisible by kv heads"):
        ops.areno_varlen_causal_attention(q[:, :3], k, v, cu)
