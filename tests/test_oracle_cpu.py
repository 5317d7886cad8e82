"""Pins the CPU oracle without a GPU: every function is checked against something that is not
its own formula -- a float64 brute force, torch's SDPA, an invariant of the mathematics, the
second (plain C) restatement, or an exhaustive table."""

import math

import numpy as np
import pytest
import torch

from areno_amd import workloads
from oracle import attention_ref as ar
from oracle import quant_ref as qr


def _brute_attention(q, k, v, query_start, window_left, scale):
    """float64 triple loop over (head, query, key); q (H,Sq,D), k/v (H,Sk,D)."""
    h, sq, d = q.shape
    sk = k.shape[1]
    out = np.zeros((h, sq, d))
    qn, kn, vn = (t.double().numpy() for t in (q, k, v))
    for hh in range(h):
        for i in range(sq):
            pos = query_start + i
            keys = [p for p in range(sk) if p <= pos and (window_left < 0 or p >= pos - window_left)]
            s = np.array([float(np.dot(qn[hh, i], kn[hh, p])) * scale for p in keys])
            w = np.exp(s - s.max())
            w /= w.sum()
            for wt, p in zip(w, keys):
                out[hh, i] += wt * vn[hh, p]
    return torch.from_numpy(out)


@pytest.mark.parametrize("query_start,window_left", [(0, -1), (5, -1), (5, 3), (0, 0), (9, 100), (2, 1)])
def test_ref_attention_vs_float64_brute_force(query_start, window_left):
    g = torch.Generator().manual_seed(3)
    h, sq, d = 3, 4, 8
    sk = query_start + sq
    q, k, v = (torch.randn(h, n, d, generator=g) for n in (sq, sk, sk))
    got = ar.ref_attention(q[None], k[None], v[None], query_start, window_left, 0.37, dtype=torch.float64)[0]
    want = _brute_attention(q, k, v, query_start, window_left, 0.37)
    torch.testing.assert_close(got, want, atol=1e-12, rtol=1e-12)


def test_ref_attention_vs_sdpa_with_explicit_mask():
    g = torch.Generator().manual_seed(4)
    h, sq, sk, d, start, win = 4, 7, 19, 16, 12, 5
    q, k, v = (torch.randn(1, h, n, d, generator=g) for n in (sq, sk, sk))
    qpos = torch.arange(start, start + sq)[:, None]
    kpos = torch.arange(sk)[None, :]
    mask = (kpos <= qpos) & (kpos >= qpos - win)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=0.2)
    got = ar.ref_attention(q, k, v, start, win, 0.2)
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)
    causal = torch.nn.functional.scaled_dot_product_attention(q[:, :, :, :], k[:, :, :sq], v[:, :, :sq], is_causal=True, scale=0.2)
    torch.testing.assert_close(ar.ref_attention(q, k[:, :, :sq], v[:, :, :sq], 0, -1, 0.2), causal, atol=2e-6, rtol=1e-5)


def test_reference_dtype_flow_differs_only_by_p_rounding():
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 2, n, 32, generator=g).bfloat16() for n in (1, 40, 40))
    a = ar.ref_attention(q, k, v, 39, -1, 32**-0.5)
    b = ar.ref_attention(q, k, v, 39, -1, 32**-0.5, reference_dtype_flow=True).float()
    assert (a - b).abs().max() < 2e-2


def _tiny(kv="fp32", **kw):
    return workloads.cfg0_tiny(kv, quantize_fn=qr.quantize, **kw)


def _decode_expected(w, window_left=-1, dtype=torch.float32):
    """Oracle output after the step's own append (float caches only)."""
    kc, vc = w.k_cache.clone().float(), w.v_cache.clone().float()
    ar.ref_decode_update(w.k_update.float(), w.v_update.float(), kc, vc, w.block_table, w.cache_seqlens)
    return ar.ref_paged_decode(w.q.float(), kc, vc, w.block_table, w.cache_seqlens, window_left, w.softmax_scale, dtype=dtype)


def test_paged_decode_block_permutation_and_padding_invariance():
    w = _tiny(poison=True)  # NaN in every slot the step must not read
    base = _decode_expected(w)
    assert torch.isfinite(base).all()
    # contiguous layout: same logical sequences copied to fresh blocks in order
    bs = w.k_cache.shape[1]
    kc = torch.full_like(w.k_cache, float("nan"))
    vc = torch.full_like(w.v_cache, float("nan"))
    table = torch.zeros_like(w.block_table)
    nxt = 0
    for b in range(4):
        need = (int(w.cache_seqlens[b]) + 1 + bs - 1) // bs
        for j in range(need):
            kc[nxt], vc[nxt] = w.k_cache[w.block_table[b, j]], w.v_cache[w.block_table[b, j]]
            table[b, j] = nxt
            nxt += 1
        table[b, need:] = 127  # arbitrary valid padding id, contents NaN
    w2 = workloads.DecodeWorkload(**{**w.__dict__, "k_cache": kc, "v_cache": vc, "block_table": table})
    torch.testing.assert_close(_decode_expected(w2), base, atol=0, rtol=0)


def test_paged_decode_gqa_equals_mha_on_repeated_kv():
    w = _tiny()
    base = _decode_expected(w)
    kc, vc = w.k_cache.clone(), w.v_cache.clone()
    ar.ref_decode_update(w.k_update, w.v_update, kc, vc, w.block_table, w.cache_seqlens)
    kc4, vc4 = kc.repeat_interleave(4, dim=2), vc.repeat_interleave(4, dim=2)
    mha = ar.ref_paged_decode(w.q, kc4, vc4, w.block_table, w.cache_seqlens, -1, w.softmax_scale)
    torch.testing.assert_close(mha, base, atol=0, rtol=0)


def test_paged_decode_special_cases():
    w = _tiny()
    lens = w.cache_seqlens.clone()
    # window >= L is no window; window 0 returns the new token's V
    torch.testing.assert_close(_decode_expected(w, window_left=10_000), _decode_expected(w), atol=0, rtol=0)
    out0 = _decode_expected(w, window_left=0)
    want = w.v_update.repeat_interleave(4, dim=1)
    torch.testing.assert_close(out0, want, atol=1e-6, rtol=1e-6)
    # L = 0: only the appended token exists
    w.cache_seqlens = torch.zeros_like(lens)
    torch.testing.assert_close(_decode_expected(w), want, atol=1e-6, rtol=1e-6)
    # all keys equal -> uniform weights -> mean of V
    w.cache_seqlens = lens
    w.k_cache[:] = 0.25
    w.k_update[:] = 0.25
    out = _decode_expected(w, dtype=torch.float64)
    for b in range(4):
        n = int(lens[b]) + 1
        vc = w.v_cache.clone()
        ar.ref_decode_update(w.k_update, w.v_update, w.k_cache.clone(), vc, w.block_table, w.cache_seqlens)
        rows = ar.gather_paged(vc, w.block_table[b], n).double().mean(0)
        torch.testing.assert_close(out[b], rows.repeat_interleave(4, dim=0), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("num_splits", [1, 2, 8, 64])
@pytest.mark.parametrize("window_left", [-1, 40])
def test_native_c_restatement_matches_torch_restatement(native_oracle, num_splits, window_left):
    w = _tiny()
    want = _decode_expected(w, window_left=window_left)
    kc, vc = w.k_cache.clone(), w.v_cache.clone()
    got = native_oracle.native_paged_decode(
        w.q, w.k_update, w.v_update, kc, vc, w.block_table, w.cache_seqlens, window_left, num_splits, w.softmax_scale
    )
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)
    # the append landed where the torch restatement puts it, and nowhere else
    kc2, vc2 = w.k_cache.clone(), w.v_cache.clone()
    ar.ref_decode_update(w.k_update, w.v_update, kc2, vc2, w.block_table, w.cache_seqlens)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)


def test_native_c_empty_splits_are_skipped(native_oracle):
    w = _tiny()
    kc, vc = w.k_cache.clone(), w.v_cache.clone()
    ar.ref_decode_update(w.k_update, w.v_update, kc, vc, w.block_table, w.cache_seqlens)
    sm, sl, sa = native_oracle.native_paged_decode_partials(w.q, kc, vc, w.block_table, w.cache_seqlens, 10, 8, w.softmax_scale)
    # an 11-key window inside >= 18 keys leaves most of the 8 splits without keys: (m, l) = (-inf, 0)
    empty = sl == 0
    assert empty.any() and torch.isinf(sm[empty]).all() and (sa[empty] == 0).all()
    want = ar.ref_paged_decode(w.q, kc, vc, w.block_table, w.cache_seqlens, 10, w.softmax_scale)
    torch.testing.assert_close(native_oracle.native_reduce(sm, sl, sa).view_as(want), want, atol=2e-6, rtol=1e-5)


def _varlen_case(seed=7, lens=(5, 1, 17, 0, 9), hq=4, hkv=2, d=16):
    g = torch.Generator().manual_seed(seed)
    t = sum(lens)
    q = torch.randn(t, hq, d, generator=g)
    k = torch.randn(t, hkv, d, generator=g)
    v = torch.randn(t, hkv, d, generator=g)
    cu = torch.tensor([0, *np.cumsum(lens)], dtype=torch.int32)
    return q, k, v, cu


@pytest.mark.parametrize("window_left", [-1, 0, 3])
def test_varlen_vs_per_sequence_sdpa_and_native_c(native_oracle, window_left):
    q, k, v, cu = _varlen_case()
    got = ar.ref_varlen(q, k, v, cu, window_left, 0.25)
    for s in range(len(cu) - 1):
        lo, hi = int(cu[s]), int(cu[s + 1])
        if hi == lo:
            continue
        n = hi - lo
        i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
        mask = (j <= i) & ((j >= i - window_left) if window_left >= 0 else True)
        kk = k[lo:hi].repeat_interleave(2, dim=1).transpose(0, 1)[None]
        vv = v[lo:hi].repeat_interleave(2, dim=1).transpose(0, 1)[None]
        want = torch.nn.functional.scaled_dot_product_attention(q[lo:hi].transpose(0, 1)[None], kk, vv, attn_mask=mask, scale=0.25)
        torch.testing.assert_close(got[lo:hi], want[0].transpose(0, 1), atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(native_oracle.native_varlen(q, k, v, cu, window_left, 0.25), got, atol=2e-6, rtol=1e-5)


def _paged_from_packed(k, v, cu, ctx_k, ctx_v, bs=4):
    """Build a paged cache holding ctx tokens then the new tokens of every sequence."""
    nseq = len(cu) - 1
    hkv, d = k.shape[1], k.shape[2]
    rows = []
    nb = 0
    for s in range(nseq):
        n = int(cu[s + 1] - cu[s]) + ctx_k[s].shape[0]
        rows.append(list(range(nb, nb + max(1, math.ceil(n / bs)))))
        nb += len(rows[-1])
    perm = torch.randperm(nb + 3, generator=torch.Generator().manual_seed(1))
    width = max(len(r) for r in rows)
    table = torch.zeros(nseq, width, dtype=torch.int32)
    kc = torch.full((nb + 3, bs, hkv, d), float("nan"))
    vc = torch.full((nb + 3, bs, hkv, d), float("nan"))
    for s, r in enumerate(rows):
        ids = perm[torch.tensor(r)]
        table[s, : len(r)] = ids.int()
        table[s, len(r) :] = ids[-1].int()
        kk = torch.cat([ctx_k[s], k[int(cu[s]) : int(cu[s + 1])]])
        vv = torch.cat([ctx_v[s], v[int(cu[s]) : int(cu[s + 1])]])
        for p in range(kk.shape[0]):
            kc[ids[p // bs], p % bs] = kk[p]
            vc[ids[p // bs], p % bs] = vv[p]
    return kc, vc, table


def test_paged_prefill_reduces_to_varlen_and_to_decode():
    q, k, v, cu = _varlen_case(lens=(5, 1, 17, 3, 9))
    nseq = len(cu) - 1
    empty = [torch.zeros(0, 2, 16)] * nseq
    kc, vc, table = _paged_from_packed(k, v, cu, empty, empty)
    zero_ctx = torch.zeros(nseq, dtype=torch.int32)
    got = ar.ref_paged_varlen_prefill(q, kc, vc, table, cu, zero_ctx, -1, 0.25)
    torch.testing.assert_close(got, ar.ref_varlen(q, k, v, cu, -1, 0.25), atol=1e-6, rtol=1e-6)
    # one new token per sequence on top of a context == paged decode with cache_seqlens = ctx
    g = torch.Generator().manual_seed(11)
    ctx_lens = torch.tensor([6, 0, 13, 4, 9], dtype=torch.int32)
    ctx_k = [torch.randn(int(n), 2, 16, generator=g) for n in ctx_lens]
    ctx_v = [torch.randn(int(n), 2, 16, generator=g) for n in ctx_lens]
    cu1 = torch.arange(nseq + 1, dtype=torch.int32)
    kc, vc, table = _paged_from_packed(k[:nseq], v[:nseq], cu1, ctx_k, ctx_v)
    pre = ar.ref_paged_varlen_prefill(q[:nseq], kc, vc, table, cu1, ctx_lens, 3, 0.25)
    dec = ar.ref_paged_decode(q[:nseq], kc, vc, table, ctx_lens, 3, 0.25)
    torch.testing.assert_close(pre, dec, atol=1e-6, rtol=1e-6)


def test_cache_write_touches_exactly_the_addressed_rows():
    g = torch.Generator().manual_seed(2)
    kc, vc = torch.randn(6, 4, 2, 8, generator=g), torch.randn(6, 4, 2, 8, generator=g)
    k, v = torch.randn(5, 2, 8, generator=g), torch.randn(5, 2, 6, generator=g)  # V narrower: zero padded
    ids = torch.tensor([3, 3, 0, 5, 1])
    offs = torch.tensor([0, 3, 2, 1, 1])
    k0, v0 = kc.clone(), vc.clone()
    ar.ref_cache_write(k, v, kc, vc, ids, offs)
    touched = torch.zeros(6, 4, dtype=torch.bool)
    touched[ids, offs] = True
    assert torch.equal(kc[~touched], k0[~touched]) and torch.equal(vc[~touched], v0[~touched])
    for t in range(5):
        assert torch.equal(kc[ids[t], offs[t]], k[t])
        assert torch.equal(vc[ids[t], offs[t], :, :6], v[t]) and (vc[ids[t], offs[t], :, 6:] == 0).all()


# ---- quantizers ---------------------------------------------------------------------------------

def _quant_inputs():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(64, 4, 128, generator=g)
    x[torch.rand(x.shape, generator=g) < 0.01] *= 8
    x[3] = 0  # zero rows
    x[5] *= 1e-9  # scale underflows fp16 -> scale 1, codes 0
    x[7] *= 3e4
    return x.bfloat16()


def test_int8_quantizer_vs_float64_brute_force_and_bounds():
    x = _quant_inputs()
    codes, scales = qr.quantize_int8(x)
    assert codes.dtype == torch.int8 and scales.dtype == torch.float16
    xf = x.float().numpy().astype(np.float64)
    amax = np.abs(xf).max(-1)
    s = np.minimum((amax.astype(np.float32) / np.float32(127)), np.float32(65504)).astype(np.float16)
    s = np.where(s == 0, np.float16(1), s)
    want = np.clip(np.rint((xf.astype(np.float32) / s.astype(np.float32)[..., None])), -127, 127).astype(np.int8)
    assert np.array_equal(codes.numpy(), want) and np.array_equal(scales.numpy(), s)
    xhat = qr.dequantize(codes, scales)
    sf = scales.float()
    normal = (amax > 1e-4) & (amax / 127 < 65504)
    err = (x.float() - xhat).abs().amax(-1)
    assert (err[torch.from_numpy(normal)] <= sf[torch.from_numpy(normal)] * 0.5 * 1.01 + 1e-30).all()
    top = codes.abs().amax(-1)[torch.from_numpy(normal)]
    assert ((top == 127) | (top == 126)).all()
    assert (codes[3] == 0).all() and (scales[3] == 1).all() and (codes[5] == 0).all()


def test_fp8_table_and_quantizer_vs_bit_layout_brute_force():
    table = qr.e4m3fn_decode_table()
    torch_table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    assert np.array_equal(np.isnan(table), np.isnan(torch_table))
    assert np.array_equal(table[~np.isnan(table)], torch_table[~np.isnan(table)])
    assert np.nanmax(table) == 448.0
    x = _quant_inputs()
    codes, scales = qr.quantize_fp8(x)
    assert codes.dtype == torch.float8_e4m3fn and scales.dtype == torch.float32
    xf = x.float()
    s = (xf.abs().amax(-1) / 448.0)
    s = torch.where(s == 0, torch.ones_like(s), s)
    y = torch.clamp(xf / s[..., None], -448, 448).numpy().astype(np.float64)
    want = qr.e4m3fn_encode_bruteforce(y)
    got = codes.view(torch.uint8).numpy()
    # -0 and +0 are the same value; compare decoded values and, away from zero, the bytes
    assert np.array_equal(table[got], table[want])
    nz = table[want] != 0
    assert np.array_equal(got[nz], want[nz])
    assert not np.isnan(table[got]).any()
    xhat = qr.dequantize(codes, scales)
    rel = ((xf - xhat).abs() / xf.abs().clamp_min(1e-30))[xf.abs() > (s[..., None] * 2**-6)]
    assert rel.max() <= 2**-4 + 1e-6  # 3 mantissa bits: half an ulp is 1/16 relative


def test_quantized_cache_write_and_decode_addresses():
    w = workloads.cfg0_tiny("int8", quantize_fn=qr.quantize)
    ids, offs = qr.decode_addresses(w.block_table, w.cache_seqlens, 16)
    kc0, ks0 = w.k_cache.clone(), w.k_scale.clone()
    qr.ref_quantized_cache_write(w.k_update, w.v_update, w.k_cache, w.v_cache, w.k_scale, w.v_scale, ids, offs)
    codes, scales = qr.quantize_int8(w.k_update)
    for b in range(4):
        pos = int(w.cache_seqlens[b])
        blk = int(w.block_table[b, pos // 16])
        assert torch.equal(w.k_cache[blk, pos % 16], codes[b]) and torch.equal(w.k_scale[blk, pos % 16], scales[b])
    touched = torch.zeros(128, 16, dtype=torch.bool)
    touched[ids, offs] = True
    assert torch.equal(w.k_cache[~touched], kc0[~touched]) and torch.equal(w.k_scale[~touched], ks0[~touched])


def test_workload_generators_are_deterministic_and_well_formed():
    a, b = _tiny("bf16"), _tiny("bf16")
    assert torch.equal(a.block_table, b.block_table) and torch.equal(a.cache_seqlens, b.cache_seqlens)
    assert torch.equal(a.k_cache.view(torch.int16), b.k_cache.view(torch.int16))
    assert a.block_table.shape == (4, 19) and a.k_cache.shape == (128, 16, 2, 64)
    assert 17 <= int(a.cache_seqlens.min()) and int(a.cache_seqlens.max()) <= 300
    # live blocks are unique across sequences
    used = []
    for r in range(4):
        used += a.block_table[r, : (int(a.cache_seqlens[r]) + 16) // 16].tolist()
    assert len(used) == len(set(used))
    w = workloads.cfg3_rollout("fp8", prompts=2, samples=3, prefix_lo=40, prefix_hi=60, median=30.0, cap=100, quantize_fn=qr.quantize)
    shared = int(w.block_table[0, 0])
    assert all(int(w.block_table[j, 0]) == shared for j in range(3)) and int(w.block_table[3, 0]) != shared
    assert w.unique_tokens < w.logical_tokens
    p = workloads.cfg4_prefill("fp8", seqs=3, new_hi=9, ctx_hi=40, quantize_fn=qr.quantize)
    assert p.q.shape[0] == int(p.cu_seqlens_q[-1]) == p.cache_block_ids.numel()
    assert p.flops() > 0
