"""Backward of the varlen and dense ops vs autograd through the CPU oracle's forward (the reference's contract:
``areno/accel/attention.py:104-118,170-183`` call native backward kernels, ``csrc/attention.cu:244-524``, which return
fp32 gradients cast to the inputs' dtypes).

Bar: the gradients are sums of 16-bit inputs accumulated in fp32 and cast back to the input dtype, so they are compared
relative to the largest gradient of the tensor: 3e-2 for bf16, 1e-2 for fp16 (one or two units of the output
format's rounding at that magnitude, plus the rounding of the saved output that both this build and the reference
use for dO . O), 1e-4 for fp32."""

import pytest
import torch

from areno_amd.accel import attention as ops
from oracle import attention_ref as ar
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu

REL = {torch.bfloat16: 3e-2, torch.float16: 1e-2, torch.float32: 1e-4}


def _close(got, want, rel, what):
    got, want = got.detach().cpu().float(), want.detach().float()
    assert torch.isfinite(got).all(), f"{what}: non-finite gradient"
    err = (got - want).abs().max().item()
    bound = rel * max(want.abs().max().item(), 1e-3)
    assert err <= bound, f"{what}: max-abs {err:.4g} > {bound:.4g}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("window_left", [None, 0, 9])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (6, 3, 128), (4, 4, 192), (4, 1, 256), (4, 4, 80), (4, 1, 96), (2, 1, 8), (6, 2, 200)])
def test_varlen_backward(dtype, window_left, hq, hkv, d):
    g = torch.Generator().manual_seed(hq * 17 + d)
    lens = [5, 1, 70, 0, 33]
    t = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q = torch.randn(t, hq, d, generator=g).to(dtype)
    k = torch.randn(t, hkv, d, generator=g).to(dtype)
    v = torch.randn(t, hkv, d, generator=g).to(dtype)
    go = torch.randn(t, hq, d, generator=g).to(dtype)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = ops.areno_varlen_causal_attention(qd, kd, vd, cu.to(DEV), window_left=window_left)
    assert out.requires_grad
    out.backward(go.to(DEV))
    qf, kf, vf = (x.float().requires_grad_(True) for x in (q, k, v))
    want = ar.ref_varlen(qf, kf, vf, cu, ar.window_left_arg(window_left), d**-0.5)
    want.backward(go.float())
    for got, ref, name in ((qd.grad, qf.grad, "dq"), (kd.grad, kf.grad, "dk"), (vd.grad, vf.grad, "dv")):
        assert got.dtype == dtype and got.shape == ref.shape
        _close(got, ref, REL[dtype], f"{name} {dtype} d={d} window={window_left}")


@pytest.mark.parametrize("last", [129, 161])
@pytest.mark.parametrize("parts,dq_rows", [("1", "16"), ("2", "32"), ("4", "16"), ("4", "32")])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,window_left", [(8, 2, 128, None), (4, 4, 64, None), (6, 1, 64, 40), (4, 2, 128, 200), (2, 1, 128, 0)])
def test_varlen_backward_long_sequences_on_the_matrix_core_kernels(dtype, hq, hkv, d, window_left, parts, dq_rows, last, monkeypatch):
    """16-bit inputs at head dims 64 / 128 take the matrix-core backward: sequences longer than its blocks of 64 rows
    and tiles of 32, blocks that hold several sequences (and empty ones), query groups, windows shorter and longer
    than a tile.  The dkv kernel in each of its shapes: key blocks of 64 rows with the stream of query tiles in one
    part or split over two, key blocks of 32 rows with four parts (the library reads the variable at every launch;
    left alone it picks by the size of the launch).  The last sequence's length makes the number of 32-row blocks
    even (1 327 tokens: every block has a partner in the four-part shape's pairs) or odd (1 359: the middle one has
    none)."""
    monkeypatch.setenv("ARENO_BACKWARD_PARTS", parts)
    monkeypatch.setenv("ARENO_BACKWARD_DQ_ROWS", dq_rows)  # the dq kernel with 16 and with 32 query rows per wave
    g = torch.Generator().manual_seed(hq * 31 + d)
    lens = [300, 1, 0, 700, 5, 63, 64, 65, last]
    t = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    q = torch.randn(t, hq, d, generator=g).to(dtype)
    k = torch.randn(t, hkv, d, generator=g).to(dtype)
    v = torch.randn(t, hkv, d, generator=g).to(dtype)
    go = torch.randn(t, hq, d, generator=g).to(dtype)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    ops.areno_varlen_causal_attention(qd, kd, vd, cu.to(DEV), window_left=window_left).backward(go.to(DEV))
    qf, kf, vf = (x.float().requires_grad_(True) for x in (q, k, v))
    ar.ref_varlen(qf, kf, vf, cu, ar.window_left_arg(window_left), d**-0.5).backward(go.float())
    for got, ref, name in ((qd.grad, qf.grad, "dq"), (kd.grad, kf.grad, "dk"), (vd.grad, vf.grad, "dv")):
        _close(got, ref, REL[dtype], f"{name} {dtype} {hq}/{hkv} d={d} window={window_left}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("query_start,window_left", [(0, None), (7, None), (3, 5)])
def test_dense_backward(dtype, query_start, window_left):
    g = torch.Generator().manual_seed(11 + query_start)
    b, h, sq, d = 3, 4, 21, 64
    sk = query_start + sq + 4  # keys behind the last query's position exist and must get zero gradient
    q = torch.randn(b, h, sq, d, generator=g).to(dtype)
    k = torch.randn(b, h, sk, d, generator=g).to(dtype)
    v = torch.randn(b, h, sk, d, generator=g).to(dtype)
    go = torch.randn(b, h, sq, d, generator=g).to(dtype)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = ops.areno_causal_attention(qd, kd, vd, query_start=query_start, window_left=window_left)
    out.backward(go.to(DEV))
    qf, kf, vf = (x.float().requires_grad_(True) for x in (q, k, v))
    want = ar.ref_attention(qf, kf, vf, query_start, ar.window_left_arg(window_left), d**-0.5)
    want.backward(go.float())
    for got, ref, name in ((qd.grad, qf.grad, "dq"), (kd.grad, kf.grad, "dk"), (vd.grad, vf.grad, "dv")):
        _close(got, ref, REL[dtype], f"dense {name} {dtype} start={query_start} window={window_left}")
    assert float(kd.grad[:, :, query_start + sq :].abs().max()) == 0.0


def test_backward_is_deterministic_and_refuses_other_head_dims():
    g = torch.Generator().manual_seed(2)
    cu = torch.tensor([0, 40, 90], dtype=torch.int32, device=DEV)
    q, k, v, go = (torch.randn(90, h, 128, generator=g).to(torch.bfloat16).to(DEV) for h in (8, 2, 2, 8))
    grads = []
    for _ in range(2):
        qd, kd, vd = (x.clone().requires_grad_(True) for x in (q, k, v))
        ops.areno_varlen_causal_attention(qd, kd, vd, cu).backward(go)
        grads.append((qd.grad, kd.grad, vd.grad))
    for a, b_ in zip(*grads):
        assert torch.equal(a, b_), "no atomics: two runs must agree bit for bit"
    # head dims the backward kernels do not cover (not a multiple of 8, or above 256) are refused by name
    for d in (20, 264):
        qx = torch.randn(10, 2, d, device=DEV, dtype=torch.float32, requires_grad=True)
        cux = torch.tensor([0, 10], dtype=torch.int32, device=DEV)
        out = ops.areno_varlen_causal_attention(qx, qx.detach(), qx.detach(), cux)
        with pytest.raises(RuntimeError, match=f"head_dim {d}"):
            out.sum().backward()


@pytest.mark.parametrize("kv,window_left", [("bf16", None), ("bf16", 11), ("fp32", None), ("int8", None)])
def test_decode_backward_recomputes_like_the_reference(kv, window_left):
    """The decode op under autograd (``_ArenoPagedCausalAttentionDecode.backward``, areno/accel/attention.py:245-264 in
    the reference): gradients of q and of the cache tensors as they stand after the append, none for the update rows;
    compared with autograd through the CPU oracle's decode on the same (appended) cache.  Quantized caches (this
    build's own) give a gradient for q only."""
    from areno_amd import workloads
    from tests.gpu_util import dequant_cpu, gpu_quantize

    act = torch.float32 if kv == "fp32" else torch.bfloat16
    lengths = torch.tensor([0, 5, 16, 37, 70])
    w = workloads.make_decode_workload("decode-backward", seed=61, batch=5, hq=8, hkv=2, d=64, bs=16, kv=kv, lengths=lengths,
                                       device=DEV, act_dtype=act, quantize_fn=gpu_quantize, pool_slack=0.5)  # fmt: skip
    q = w.q.clone().requires_grad_(True)
    quantized = w.k_scale is not None
    kc, vc = w.k_cache, w.v_cache
    if not quantized:
        kc, vc = kc.clone().requires_grad_(True), vc.clone().requires_grad_(True)
    out = ops.areno_paged_causal_attention_decode(q, w.k_update, w.v_update, kc, vc, w.block_table, w.cache_seqlens,
                                                  window_left=window_left, softmax_scale=w.softmax_scale,
                                                  k_scale=w.k_scale, v_scale=w.v_scale)  # fmt: skip
    assert out.requires_grad
    g = torch.Generator().manual_seed(9)
    grad_out = torch.randn(out.shape, generator=g).to(out.dtype)
    out.backward(grad_out.to(DEV))

    # the oracle on the cache after the append, in fp32 on the CPU
    k_ref, v_ref = (dequant_cpu(kc.detach(), w.k_scale), dequant_cpu(vc.detach(), w.v_scale))
    q_ref = w.q.detach().cpu().float().requires_grad_(True)
    k_ref, v_ref = k_ref.requires_grad_(True), v_ref.requires_grad_(True)
    want = ar.ref_paged_decode(q_ref, k_ref, v_ref, w.block_table.cpu(), w.cache_seqlens.cpu(),
                               -1 if window_left is None else window_left, w.softmax_scale)  # fmt: skip
    want.backward(grad_out.float())
    rel = REL[act]
    _close(q.grad, q_ref.grad, rel, "dq")
    if quantized:
        assert w.k_update.grad is None
    else:
        _close(kc.grad, k_ref.grad, rel, "dk_cache")
        _close(vc.grad, v_ref.grad, rel, "dv_cache")
        live = set(w.block_table.cpu().flatten().tolist())
        untouched = [b for b in range(kc.shape[0]) if b not in live]
        assert float(kc.grad[untouched].abs().max()) == 0.0, "pages no row lists must get no gradient"


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float16, 64), (torch.bfloat16, 96), (torch.float32, 64)])
def test_gradients_in_the_input_dtype_are_the_fp32_gradients_rounded_once(dtype, d):
    """The extension's backward with fp32 gradients (the reference launchers' contract) and with gradients in the
    inputs' dtype (what the autograd functions ask for): the second is the first cast, bit for bit, on the
    matrix-core kernels (head dims 64 / 128) and on the vector-ALU ones (96; fp32 inputs)."""
    from areno_amd.accel.attention import _extension

    g = torch.Generator().manual_seed(d)
    lens = [70, 1, 129, 300]
    t, hq, hkv = sum(lens), 6, 2
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    q, go = (torch.randn(t, hq, d, generator=g).to(dtype).to(DEV) for _ in range(2))
    k, v = (torch.randn(t, hkv, d, generator=g).to(dtype).to(DEV) for _ in range(2))
    out = ops.areno_varlen_causal_attention(q, k, v, cu)
    wide = _extension().areno_attention_backward(go, q, k, v, out, cu, None, None, -1, d**-0.5, False)
    typed = _extension().areno_attention_backward(go, q, k, v, out, cu, None, None, -1, d**-0.5, True)
    for a, b, name in zip(wide, typed, ("dq", "dk", "dv")):
        assert a.dtype == torch.float32 and b.dtype == dtype
        assert torch.equal(a.to(dtype), b), f"{name} {dtype} d={d}"
