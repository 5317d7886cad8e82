"""HIP kernels against the committed golden vectors (no oracle run on the box for these)."""

import os

import numpy as np
import pytest
import torch

from areno_amd import workloads
from areno_amd.accel import attention as ops
from oracle import quant_ref as qr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_vectors.npz"))


def _to(w, dev):
    for name in ("q", "k_update", "v_update", "k_cache", "v_cache", "k_scale", "v_scale", "block_table", "cache_seqlens"):
        t = getattr(w, name)
        if t is not None:
            setattr(w, name, t.to(dev))
    return w


@pytest.mark.parametrize("kv,tol", [("fp32", 2e-2), ("bf16", 2e-2), ("int8", 5e-2), ("fp8", 5e-2)])
@pytest.mark.parametrize("window", [-1, 40])
def test_decode_against_golden(kv, tol, window):
    # inputs are generated on the CPU (seeded, machine independent) and quantized by the oracle, then moved over
    w = _to(workloads.cfg0_tiny(kv, quantize_fn=qr.quantize), DEV)
    out = ops.areno_paged_causal_attention_decode(
        w.q, w.k_update, w.v_update, w.k_cache, w.v_cache, w.block_table, w.cache_seqlens,
        window_left=None if window < 0 else window, softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale,
    )  # fmt: skip
    err = np.abs(out.float().cpu().numpy() - GOLD[f"cfg0_decode_{kv}_w{window}"])
    assert err.max() <= tol, f"{kv} window {window}: max-abs {err.max()}"


def test_quantizer_against_golden_bit_exact():
    g = torch.Generator().manual_seed(4242)
    x = (torch.randn(8, 2, 64, generator=g) * torch.tensor([0.01, 1.0, 30.0, 1e-6]).repeat(2).view(8, 1, 1)).bfloat16()
    ids = torch.arange(8, device=DEV)
    for cdt, sdt, ck, sk in ((torch.int8, torch.float16, "quant_int8_codes", "quant_int8_scales"),
                             (torch.float8_e4m3fn, torch.float32, "quant_fp8_codes", "quant_fp8_scales")):  # fmt: skip
        kc = torch.zeros(8, 1, 2, 64, dtype=torch.uint8, device=DEV).view(cdt)
        vc = torch.zeros_like(kc)
        ks = torch.zeros(8, 1, 2, dtype=sdt, device=DEV)
        vs = torch.zeros_like(ks)
        ops.areno_paged_cache_write(x.to(DEV), x.to(DEV), kc, vc, ids, torch.zeros_like(ids), k_scale=ks, v_scale=vs)
        got = kc.view(torch.uint8).cpu().numpy().reshape(8, 2, 64)
        want = GOLD[ck].view(np.uint8)
        if cdt == torch.float8_e4m3fn:  # +0 / -0
            got, want = np.where(got == 0x80, 0, got), np.where(want == 0x80, 0, want)
        assert np.array_equal(got, want)
        assert np.array_equal(ks.cpu().numpy().reshape(8, 2), GOLD[sk])


def test_prefill_against_golden():
    p = workloads.make_prefill_workload("golden-prefill", seed=77, new_lens=torch.tensor([9, 1, 20]), ctx_lens=torch.tensor([37, 0, 64]),
                                        hq=8, hkv=2, d=64, bs=16, kv="fp8", quantize_fn=qr.quantize)
    out = ops.areno_paged_varlen_causal_attention(
        p.q.to(DEV), p.k_cache.to(DEV), p.v_cache.to(DEV), p.block_table.to(DEV), p.cu_seqlens_q.to(DEV),
        p.context_lens.to(DEV), softmax_scale=p.softmax_scale, k_scale=p.k_scale.to(DEV), v_scale=p.v_scale.to(DEV),
    )  # fmt: skip
    err = np.abs(out.float().cpu().numpy() - GOLD["prefill_fp8"])
    assert err.max() <= 5e-2
