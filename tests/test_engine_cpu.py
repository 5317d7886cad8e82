"""Engine-side glue without a GPU: cache geometry, metadata carrier, argument checks of the backend module
(the checks mirror areno/engine/layers/attention_backend/infer.py:73-75,106-117,180-185 in the reference)."""

import pytest
import torch

from areno_amd.engine import HipInferBackend, InferMeta, allocate_kv_caches, build_infer_attention_backend
from areno_amd.engine import kv_cache_bytes_per_token
from areno_amd.engine.attention_backend import _window_left, pad_last_dim


def test_allocate_kv_caches_geometry_and_dtypes():
    plain = allocate_kv_caches(3, 9, 16, 2, 64, "cpu", torch.bfloat16)
    assert len(plain) == 3 and not plain[0].quantized
    assert plain[0].k_cache.shape == (9, 16, 2, 64) and plain[0].v_cache.dtype == torch.bfloat16
    assert plain[0].as_tuple()[0] is plain[0].k_cache
    q8 = allocate_kv_caches(1, 5, 16, 4, 128, "cpu", torch.bfloat16, "int8")[0]
    assert q8.k_cache.dtype == torch.int8 and q8.k_scale.dtype == torch.float16 and q8.k_scale.shape == (5, 16, 4)
    assert float(q8.v_scale.min()) == 1.0 and int(q8.v_cache.abs().max()) == 0  # unwritten slots decode to 0.0
    f8 = allocate_kv_caches(1, 5, 16, 4, 128, "cpu", torch.float16, "fp8")[0]
    assert f8.v_cache.dtype == torch.float8_e4m3fn and f8.v_scale.dtype == torch.float32
    with pytest.raises(ValueError, match="kv_cache_dtype"):
        allocate_kv_caches(1, 5, 16, 4, 128, "cpu", torch.float16, "int4")
    with pytest.raises(ValueError, match="positive"):
        allocate_kv_caches(1, 0, 16, 4, 128, "cpu", torch.float16)


def test_bytes_per_token_match_the_kernel_accounting():
    # the per-token figures the decode roofline uses: 2048 B bf16 (Hkv 4, D 128), 1040 B int8, 2112 B fp8 (Hkv 8)
    assert kv_cache_bytes_per_token(4, 128, torch.bfloat16) == 2048
    assert kv_cache_bytes_per_token(4, 128, torch.bfloat16, "int8") == 1040
    assert kv_cache_bytes_per_token(8, 128, torch.bfloat16, "fp8") == 2112


def test_window_and_padding_helpers():
    assert _window_left(None) is None and _window_left((-1, -1)) is None and _window_left((7, 0)) == 7
    with pytest.raises(ValueError, match="right window 0"):
        _window_left((7, 1))
    x = torch.ones(2, 3, 5)
    assert pad_last_dim(x, 5) is x
    y = pad_last_dim(x, 8)
    assert y.shape == (2, 3, 8) and float(y[..., 5:].abs().sum()) == 0.0
    with pytest.raises(ValueError, match="cannot fit"):
        pad_last_dim(x, 4)


def test_backend_argument_checks_come_before_any_kernel():
    backend = build_infer_attention_backend("native")
    assert isinstance(backend, HipInferBackend)
    with pytest.raises(ValueError, match="attn_backend"):
        build_infer_attention_backend("triton")
    q = torch.zeros(1, 4, 8, 64)
    k = torch.zeros(1, 4, 2, 64)
    cache = torch.zeros(3, 16, 2, 64)
    with pytest.raises(ValueError, match="requires cu_seqlens"):
        backend(q, k, k, cache, cache, InferMeta(mode="prefill"))
    meta = InferMeta(mode="prefill", cu_seqlens=torch.tensor([0, 4], dtype=torch.int32), max_seqlen=4,
                     block_table=torch.zeros(1, 1, dtype=torch.int32))  # fmt: skip
    with pytest.raises(ValueError, match="cache_block_ids"):
        backend(q, k, k, cache, cache, meta)
    with pytest.raises(ValueError, match="requires cache_seqlens"):
        backend(q, k, k, cache, cache, InferMeta(mode="decode"))
    dec = InferMeta(mode="decode", cache_seqlens=torch.zeros(4, dtype=torch.int64),
                    block_table=torch.zeros(4, 1, dtype=torch.int32))  # fmt: skip
    with pytest.raises(ValueError, match="update_cache=True"):
        backend(q, k, k, cache, cache, dec, update_cache=False)
    with pytest.raises(ValueError, match="int32 cache_seqlens"):
        backend(q, k, k, cache, cache, dec)
    with pytest.raises(ValueError, match="given together"):
        backend(q, k, k, cache, cache, dec, k_scale=torch.ones(3, 16, 2))
    with pytest.raises(ValueError, match="unsupported inference mode"):
        backend(q, k, k, cache, cache, InferMeta(mode="train"))  # type: ignore[arg-type]
