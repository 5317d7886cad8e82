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
