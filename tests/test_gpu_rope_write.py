"""Fused QK RMSNorm + rotary + quantizing cache write vs the CPU oracle (the layer's steps in front of the path,
areno/engine/layers/attention.py:90-96 and attention_backend/infer.py:245-263 in the reference).

Bars: q / k after norm and rotary within three units in the last place (of the row's magnitude, in the activation
dtype) of the oracle: the reciprocal square root differs in its last bit between the GPU instruction and the CPU,
which can move the normalised value and each rotary product by one unit; without a norm the rotary arithmetic is
bit-exact.  The pages must hold bit for bit what the stand-alone cache write stores for the op's own
k output and for v."""

import pytest
import torch

from areno_amd.accel import attention as ops
from areno_amd.engine import allocate_kv_caches
from oracle import rope_ref as rr
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _inputs(t, hq, hkv, d, dtype, seed, max_pos=4096):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(t, hq, d, generator=g) * 2).to(dtype)
    k = (torch.randn(t, hkv, d, generator=g) * 2).to(dtype)
    v = torch.randn(t, hkv, d, generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (t,), generator=g)
    pos[0] = 0
    cos, sin = rr.rope_tables(d, max_pos, 1_000_000.0)
    qw = torch.rand(d, generator=g) + 0.5
    kw = torch.rand(d, generator=g) + 0.5
    return q, k, v, pos, cos, sin, qw, kw


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (28, 4, 128), (4, 4, 256), (2, 2, 512), (1, 1, 64), (3, 1, 128), (32, 8, 128), (2, 1, 64), (6, 2, 128)])
@pytest.mark.parametrize("norm", [True, False])
def test_norm_rope_outputs(dtype, hq, hkv, d, norm):
    q, k, v, pos, cos, sin, qw, kw = _inputs(37, hq, hkv, d, dtype, seed=d + hq)
    weights = dict(q_norm_weight=qw.to(DEV), k_norm_weight=kw.to(DEV)) if norm else {}
    q_out, k_out = ops.areno_qk_norm_rope_cache_write(q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), cos.to(DEV),
                                                      sin.to(DEV), eps=1e-6, **weights)  # fmt: skip
    want_q, want_k = rr.ref_qk_norm_rope(q, k, pos, cos, sin, qw if norm else None, kw if norm else None, 1e-6)
    if norm:
        # an ulp of the normalised value moves each rotary product by an ulp; allow three in total
        for got, want, name in ((q_out, want_q, "q"), (k_out, want_k, "k")):
            err = (got.cpu().float() - want.float()).abs()
            eps = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
            scale = want.float().abs().amax(dim=-1, keepdim=True)  # rotary mixes two elements of the row
            assert float((err / (eps * scale)).max()) <= 3.0, f"{name}: beyond 3 ulp of the row magnitude"
    else:
        assert torch.equal(q_out.cpu(), want_q), "rotary without norm must be bit-exact (q)"
        assert torch.equal(k_out.cpu(), want_k), "rotary without norm must be bit-exact (k)"


@pytest.mark.parametrize("kv", ["auto", "int8", "fp8"])
def test_pages_hold_the_quantized_outputs(kv):
    t, hq, hkv, d, bs = 53, 16, 4, 128, 16
    dtype = torch.bfloat16
    q, k, v, pos, cos, sin, qw, kw = _inputs(t, hq, hkv, d, dtype, seed=7)
    nb = 8
    fused = allocate_kv_caches(1, nb, bs, hkv, d, DEV, dtype, kv)[0]
    plain = allocate_kv_caches(1, nb, bs, hkv, d, DEV, dtype, kv)[0]
    for layer in (fused, plain):  # same starting contents, so untouched slots compare equal too
        layer.k_cache.view(torch.uint8).fill_(0x11)
        layer.v_cache.view(torch.uint8).fill_(0x11)
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(nb * bs, generator=g)[:t]
    ids, offs = (slots // bs).to(DEV), (slots % bs).to(DEV)
    q_out, k_out = ops.areno_qk_norm_rope_cache_write(
        q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), cos.to(DEV), sin.to(DEV), q_norm_weight=qw.to(DEV),
        k_norm_weight=kw.to(DEV), eps=1e-6, k_cache=fused.k_cache, v_cache=fused.v_cache, cache_block_ids=ids,
        cache_block_offsets=offs, k_scale=fused.k_scale, v_scale=fused.v_scale,
    )  # fmt: skip
    ops.areno_paged_cache_write(k_out, v.to(DEV), plain.k_cache, plain.v_cache, ids, offs, k_scale=plain.k_scale,
                                v_scale=plain.v_scale)  # fmt: skip
    torch.cuda.synchronize()
    for a, b, name in ((fused.k_cache, plain.k_cache, "k"), (fused.v_cache, plain.v_cache, "v"),
                       (fused.k_scale, plain.k_scale, "k_scale"), (fused.v_scale, plain.v_scale, "v_scale")):  # fmt: skip
        if a is not None:
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{name} pages differ from the plain write"
    want_q, _ = rr.ref_qk_norm_rope(q, k, pos, cos, sin, qw, kw, 1e-6)
    err = (q_out.cpu().float() - want_q.float()).abs()
    assert float(err.max()) < 0.1


def test_token_ranges_give_what_one_launch_gives():
    """A call whose token count is past the kernel's 32-bit indexing runs as consecutive launches over token ranges;
    with the range capped at 5 tokens (the library's test hook) a 53-token call must leave the same outputs and pages,
    bit for bit, as one launch."""
    import ctypes

    from areno_amd.accel import cabi

    lib = cabi.lib()
    lib.areno_hip_debug_set_rope_tokens_per_launch.restype = ctypes.c_int64
    lib.areno_hip_debug_set_rope_tokens_per_launch.argtypes = [ctypes.c_int64]
    t, hq, hkv, d, bs, nb = 53, 16, 4, 128, 16, 8
    dtype = torch.bfloat16
    q, k, v, pos, cos, sin, qw, kw = _inputs(t, hq, hkv, d, dtype, seed=11)
    g = torch.Generator().manual_seed(4)
    slots = torch.randperm(nb * bs, generator=g)[:t]
    ids, offs = (slots // bs).to(DEV), (slots % bs).to(DEV)
    results = []
    for cap in (0, 5):
        layer = allocate_kv_caches(1, nb, bs, hkv, d, DEV, dtype, "fp8")[0]
        layer.k_cache.view(torch.uint8).fill_(0x11)
        layer.v_cache.view(torch.uint8).fill_(0x11)
        before = lib.areno_hip_debug_set_rope_tokens_per_launch(cap)
        try:
            q_out, k_out = ops.areno_qk_norm_rope_cache_write(
                q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), cos.to(DEV), sin.to(DEV), q_norm_weight=qw.to(DEV),
                k_norm_weight=kw.to(DEV), eps=1e-6, k_cache=layer.k_cache, v_cache=layer.v_cache, cache_block_ids=ids,
                cache_block_offsets=offs, k_scale=layer.k_scale, v_scale=layer.v_scale,
            )  # fmt: skip
            torch.cuda.synchronize()
        finally:
            lib.areno_hip_debug_set_rope_tokens_per_launch(before)
        results.append((q_out, k_out, layer.k_cache, layer.v_cache, layer.k_scale, layer.v_scale))
    for a, b, name in zip(results[0], results[1], ("q_out", "k_out", "k pages", "v pages", "k scales", "v scales")):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{name} differ between one launch and eleven"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (28, 4, 128), (4, 4, 256), (2, 2, 512)])
def test_prepared_rotary_rows_give_the_same_bits(dtype, hq, hkv, d):
    """areno_rope_rows prepares a step's cosines and sines once (rounded to the activation dtype, rotate_half's sign
    on the sines); every layer's fused call then takes them as rope_rows.  Outputs and pages must be what the call
    with positions and tables gives, bit for bit -- with positions outside the table (clamped by both), with and
    without the norm, and when the call runs as several launches over token ranges."""
    import ctypes

    from areno_amd.accel import cabi

    t, bs, nb = 61, 16, 8
    q, k, v, pos, cos, sin, qw, kw = _inputs(t, hq, hkv, d, dtype, seed=3 * d + hq, max_pos=512)
    pos[1], pos[2] = -5, 100_000  # clamped into the table by both paths
    rows = ops.areno_rope_rows(pos.to(DEV), cos.to(DEV), sin.to(DEV), dtype)
    assert rows.shape == (t, 2, d) and rows.dtype == torch.float32
    pc = pos.clamp(0, 511)
    assert torch.equal(rows[:, 0].cpu(), cos[pc].to(dtype).float())
    sign = torch.cat([-torch.ones(d // 2), torch.ones(d // 2)])
    assert torch.equal(rows[:, 1].cpu(), sin[pc].to(dtype).float() * sign)
    g = torch.Generator().manual_seed(9)
    slots = torch.randperm(nb * bs, generator=g)[:t]
    ids, offs = (slots // bs).to(DEV), (slots % bs).to(DEV)
    lib = cabi.lib()
    lib.areno_hip_debug_set_rope_tokens_per_launch.restype = ctypes.c_int64
    lib.areno_hip_debug_set_rope_tokens_per_launch.argtypes = [ctypes.c_int64]
    for norm, cap in ((True, 0), (False, 0), (True, 7)):
        weights = dict(q_norm_weight=qw.to(DEV), k_norm_weight=kw.to(DEV)) if norm else {}
        results = []
        for use_rows in (False, True):
            layer = allocate_kv_caches(1, nb, bs, hkv, d, DEV, dtype, "int8")[0]
            layer.k_cache.view(torch.uint8).fill_(0x11)
            layer.v_cache.view(torch.uint8).fill_(0x11)
            before = lib.areno_hip_debug_set_rope_tokens_per_launch(cap)
            try:
                q_out, k_out = ops.areno_qk_norm_rope_cache_write(
                    q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), cos.to(DEV), sin.to(DEV), eps=1e-6,
                    k_cache=layer.k_cache, v_cache=layer.v_cache, cache_block_ids=ids, cache_block_offsets=offs,
                    k_scale=layer.k_scale, v_scale=layer.v_scale, rope_rows=rows if use_rows else None, **weights,
                )  # fmt: skip
                torch.cuda.synchronize()
            finally:
                lib.areno_hip_debug_set_rope_tokens_per_launch(before)
            results.append((q_out, k_out, layer.k_cache, layer.v_cache, layer.k_scale, layer.v_scale))
        for a, b, name in zip(results[0], results[1], ("q_out", "k_out", "k pages", "v pages", "k scales", "v scales")):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{name} differ (norm={norm}, cap={cap})"


def test_argument_checks():
    q, k, v, pos, cos, sin, qw, kw = _inputs(4, 4, 2, 128, torch.bfloat16, seed=1)
    with pytest.raises(RuntimeError, match="requires CUDA"):
        ops.areno_qk_norm_rope_cache_write(q, k, v, pos, cos, sin)
    dev = [t.to(DEV) for t in (q, k, v, pos, cos, sin)]
    with pytest.raises(ValueError, match="fp16 or bf16"):
        ops.areno_qk_norm_rope_cache_write(dev[0].float(), dev[1].float(), dev[2].float(), *dev[3:])
    with pytest.raises(ValueError, match="together"):
        ops.areno_qk_norm_rope_cache_write(*dev, k_cache=torch.empty(2, 16, 2, 128, device=DEV, dtype=torch.bfloat16))
    q96 = torch.zeros(4, 4, 96, device=DEV, dtype=torch.bfloat16)
    k96 = torch.zeros(4, 2, 96, device=DEV, dtype=torch.bfloat16)
    c96 = torch.zeros(16, 96, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim"):
        ops.areno_qk_norm_rope_cache_write(q96, k96, k96, dev[3], c96, c96)
    out_q, out_k = ops.areno_qk_norm_rope_cache_write(dev[0][:0], dev[1][:0], dev[2][:0], dev[3][:0], dev[4], dev[5])
    assert out_q.shape == (0, 4, 128) and out_k.shape == (0, 2, 128)
