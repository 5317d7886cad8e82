"""Cache-write kernel: block placement and codes must be bit-exact against the oracle's closed forms."""

import pytest
import torch

from areno_amd.accel import attention as ops
from oracle import attention_ref as ar
from oracle import quant_ref as qr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(t, hkv, d, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(2, t, hkv, d, generator=g)
    x[torch.rand(x.shape, generator=g) < 0.01] *= 8
    x[:, 0] = 0
    if t > 4:
        x[:, 1] *= 1e-9
        x[:, 2] *= 3e4 if dtype != torch.float16 else 1e3  # stay finite in fp16: non-finite rows are outside the contract
        x[:, 3, :, 0] = 0.5  # exact halves after scaling exercise round-half-even
    return x[0].to(dtype), x[1].to(dtype)


def _addresses(t, nb, bs, seed=1):
    g = torch.Generator().manual_seed(seed)
    flat = torch.randperm(nb * bs, generator=g)[:t]
    return flat // bs, flat % bs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("d", [64, 128, 80, 256, 512, 192])
def test_unquantized_scatter_is_a_bit_exact_copy(dtype, d):
    t, hkv, nb, bs = 37, 4, 9, 16
    k, v = _inputs(t, hkv, d, dtype)
    ids, offs = _addresses(t, nb, bs)
    g = torch.Generator().manual_seed(5)
    kc = torch.randn(nb, bs, hkv, d, generator=g).to(dtype)
    vc = torch.randn(nb, bs, hkv, d, generator=g).to(dtype)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ar.ref_cache_write(k, v, kc_ref, vc_ref, ids, offs)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    ops.areno_paged_cache_write(k.to(DEV), v.to(DEV), kc_d, vc_d, ids.to(DEV), offs.to(DEV))
    assert torch.equal(kc_d.cpu(), kc_ref) and torch.equal(vc_d.cpu(), vc_ref)


@pytest.mark.parametrize("cache_dtype,scale_dtype", [(torch.int8, torch.float16), (torch.float8_e4m3fn, torch.float32)])
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("d", [128, 64, 256, 512, 96])
def test_quantize_and_scatter_bit_exact(cache_dtype, scale_dtype, in_dtype, d):
    # 16-bit rows of 64 / 128 / 256 / 512 elements take the writer's lane-group kernel (several rows per wave, 300 x 4
    # rows do not fill the last wave), everything else the one-row-per-wave kernel; both must give the same bits
    t, hkv, nb, bs = 300, 4, 40, 16
    k, v = _inputs(t, hkv, d, in_dtype, seed=3)
    ids, offs = _addresses(t, nb, bs, seed=4)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.uint8).view(cache_dtype)
    vc = torch.zeros_like(kc)
    kc.view(torch.uint8)[:] = 0x11
    vc.view(torch.uint8)[:] = 0x22
    ks = torch.full((nb, bs, hkv), 7.0, dtype=scale_dtype)
    vs = torch.full((nb, bs, hkv), 9.0, dtype=scale_dtype)
    ref = [t_.clone() for t_ in (kc, vc, ks, vs)]
    qr.ref_quantized_cache_write(k, v, *ref, ids, offs)
    dev = [t_.to(DEV) for t_ in (kc, vc, ks, vs)]
    ops.areno_paged_cache_write(k.to(DEV), v.to(DEV), dev[0], dev[1], ids.to(DEV), offs.to(DEV), k_scale=dev[2], v_scale=dev[3])
    for name, got, want in zip(("k codes", "v codes", "k scale", "v scale"), dev, ref):
        got = got.cpu()
        if got.dtype in (torch.int8, torch.float8_e4m3fn):
            gb, wb = got.view(torch.uint8), want.view(torch.uint8)
            if cache_dtype == torch.float8_e4m3fn:  # +0 and -0 are one value
                gb = torch.where(gb == 0x80, torch.zeros_like(gb), gb)
                wb = torch.where(wb == 0x80, torch.zeros_like(wb), wb)
            assert torch.equal(gb, wb), f"{name}: {(gb != wb).sum().item()} bytes differ"
        else:
            assert torch.equal(got, want), name


def test_fp8_encoder_exhaustive_grid():
    """Every e4m3 value, every midpoint between neighbours and values just off the midpoints."""
    table = torch.from_numpy(qr.e4m3fn_decode_table()).float()
    finite = torch.sort(table[torch.isfinite(table)]).values.unique()
    mids = (finite[1:] + finite[:-1]) / 2
    pts = torch.cat([finite, mids, torch.nextafter(mids, mids + 1), torch.nextafter(mids, mids - 1)])
    pts = pts[pts.abs() <= 448]
    pad = (-pts.numel()) % 128
    pts = torch.cat([pts, pts.new_zeros(pad)])
    x = pts.view(-1, 1, 128).clone()
    x[:, 0, 0] = 448.0  # pins every row's scale to exactly 1
    codes, scales = qr.quantize_fp8(x)
    assert (scales == 1).all()
    n = x.shape[0]
    kc = torch.zeros(n, 1, 1, 128, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(n, 1, 1, dtype=torch.float32, device=DEV)
    vs = torch.zeros_like(ks)
    ids = torch.arange(n, device=DEV)
    ops.areno_paged_cache_write(x.to(DEV), x.to(DEV), kc, vc, ids, torch.zeros_like(ids), k_scale=ks, v_scale=vs)
    assert torch.equal(kc.cpu().float().view(n, 1, 128), codes.float())
    assert (ks.cpu() == 1).all()


def test_int8_rounding_ties_and_clamp():
    x = torch.zeros(4, 1, 128)
    x[0, 0, :8] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5])  # scale = 1
    x[1, 0, :3] = torch.tensor([254.0, 1.0, 3.0])  # scale = 2: 0.5 -> 0, 1.5 -> 2
    x[2, 0, :2] = torch.tensor([1e-7, -1e-7])  # scale underflows -> 1, codes 0
    x[3, 0, :2] = torch.tensor([9e6, -9e6])  # scale clamps at 65504 -> codes clamp at +-127
    codes, scales = qr.quantize_int8(x)
    assert codes[0, 0, :8].tolist() == [127, 0, 2, 2, 0, -2, -2, 126]
    assert codes[1, 0, :3].tolist() == [127, 0, 2] and codes[3, 0, :2].tolist() == [127, -127]
    kc = torch.zeros(4, 1, 1, 128, dtype=torch.int8, device=DEV)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(4, 1, 1, dtype=torch.float16, device=DEV)
    vs = torch.zeros_like(ks)
    ids = torch.arange(4, device=DEV)
    ops.areno_paged_cache_write(x.to(DEV), x.to(DEV), kc, vc, ids, torch.zeros_like(ids), k_scale=ks, v_scale=vs)
    assert torch.equal(kc.cpu().view(4, 1, 128), codes) and torch.equal(ks.cpu().view(4, 1), scales)
    assert torch.equal(vc.cpu().view(4, 1, 128), codes)


@pytest.mark.parametrize("cache_dtype,scale_dtype", [(torch.int8, torch.float16), (torch.float8_e4m3fn, torch.float32)])
def test_quantizer_divisions_over_the_range_of_scales(cache_dtype, scale_dtype):
    """bf16 rows whose abs-max runs from 2^-120 to 2^100: the lane-group kernel divides a row by its scale through one
    shared reciprocal when the scale lies in 2^-60 .. 2^60 and by the plain division outside; both must give the
    oracle's codes, with negative zeros, exact halves and denormal elements among the values."""
    exps = [-120, -100, -70, -62, -61, -60, -59, -45, -20, -3, 0, 7, 30, 58, 59, 60, 61, 62, 70, 100]
    hkv, d, bs = 2, 128, 16
    t = len(exps) * 3
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, t, hkv, d, generator=g)
    x[torch.rand(x.shape, generator=g) < 0.05] = -0.0
    x[torch.rand(x.shape, generator=g) < 0.05] *= 2.0 ** -20
    scale = torch.tensor([2.0**e for e in exps for _ in range(3)], dtype=torch.float64).view(1, t, 1, 1)
    x = (x.double() * scale).to(torch.bfloat16)
    x[:, :, :, 0] = (448.0 * scale[..., 0]).to(torch.bfloat16)  # an abs-max of exactly 448 x 2^e: fp8 scale 2^e
    x[:, :, :, 1] = (0.5 * 2.0**-6 * scale[..., 0]).to(torch.bfloat16)  # half of fp8's smallest normal step: a tie
    k, v = x[0], x[1]
    nb = (t + bs - 1) // bs + 1
    ids, offs = _addresses(t, nb, bs, seed=8)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.uint8).view(cache_dtype)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(nb, bs, hkv, dtype=scale_dtype)
    vs = torch.zeros_like(ks)
    ref = [t_.clone() for t_ in (kc, vc, ks, vs)]
    qr.ref_quantized_cache_write(k, v, *ref, ids, offs)
    dev = [t_.to(DEV) for t_ in (kc, vc, ks, vs)]
    ops.areno_paged_cache_write(k.to(DEV), v.to(DEV), dev[0], dev[1], ids.to(DEV), offs.to(DEV), k_scale=dev[2], v_scale=dev[3])
    for name, got, want in zip(("k codes", "v codes", "k scale", "v scale"), dev, ref):
        got = got.cpu()
        if got.dtype in (torch.int8, torch.float8_e4m3fn):
            gb, wb = got.view(torch.uint8), want.view(torch.uint8)
            if cache_dtype == torch.float8_e4m3fn:  # +0 and -0 are one value
                gb = torch.where(gb == 0x80, torch.zeros_like(gb), gb)
                wb = torch.where(wb == 0x80, torch.zeros_like(wb), wb)
            bad = (gb != wb).nonzero()
            assert bad.numel() == 0, f"{name}: {bad.shape[0]} bytes differ, first at {bad[0].tolist()}"
        else:
            assert torch.equal(got, want), name


def test_out_of_pool_addresses_are_skipped_and_empty_write_is_a_noop():
    kc = torch.zeros(2, 4, 1, 64, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    k = torch.ones(3, 1, 64, dtype=torch.bfloat16, device=DEV)
    ids = torch.tensor([0, 5, -1], device=DEV)
    offs = torch.tensor([1, 0, 0], device=DEV)
    ops.areno_paged_cache_write(k, k, kc, vc, ids, offs)
    assert kc.sum().item() == 64 and kc[0, 1].sum().item() == 64
    ops.areno_paged_cache_write(k[:0], k[:0], kc, vc, ids[:0], offs[:0])
    assert kc.sum().item() == 64
