"""ctypes wrapper over ``oracle/native_kernels.c`` (TEST INFRASTRUCTURE ONLY).

``build()`` compiles the C file with gcc through ``oracle/Makefile``;
``load()`` loads an already built library and raises if it is missing.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_native.so")
_LIB: ctypes.CDLL | None = None

_F = ctypes.POINTER(ctypes.c_float)
_I = ctypes.POINTER(ctypes.c_int32)
_L = ctypes.c_int64


def build() -> str:
    subprocess.run(["make", "-B", "-C", _HERE, "liboracle_native.so"], check=True, capture_output=True)
    return _LIB_PATH


def load() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f"{_LIB_PATH} is not built; run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_paged_decode.restype = ctypes.c_int
        lib.oracle_paged_decode.argtypes = [_F, _F, _F, _F, _F, _I, _I, _F] + [_L] * 8 + [ctypes.c_float]
        lib.oracle_paged_decode_split.restype = None
        lib.oracle_paged_decode_split.argtypes = [_F, _F, _F, _I, _I, _F, _F, _F] + [_L] * 8 + [ctypes.c_float]
        lib.oracle_paged_decode_reduce.restype = None
        lib.oracle_paged_decode_reduce.argtypes = [_F, _F, _F, _F, _L, _L, _L]
        lib.oracle_varlen_forward.restype = None
        lib.oracle_varlen_forward.argtypes = [_F, _F, _F, _F, _I] + [_L] * 6 + [ctypes.c_float]
        _LIB = lib
    return _LIB


def _fp(t: torch.Tensor | None):
    if t is None:
        return ctypes.cast(None, _F)
    assert t.dtype == torch.float32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.cast(t.data_ptr(), _F)


def _ip(t: torch.Tensor):
    assert t.dtype == torch.int32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.cast(t.data_ptr(), _I)


def native_paged_decode(
    q, k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, window_left, num_splits, softmax_scale
):
    """fp32 decode op (update + split + reduce); caches (fp32) are updated in place when updates are given."""
    b, hq, d = q.shape
    out = torch.empty_like(q)
    rc = load().oracle_paged_decode(
        _fp(q), _fp(k_update), _fp(v_update), _fp(k_cache), _fp(v_cache), _ip(block_table), _ip(cache_seqlens),
        _fp(out), b, hq, k_cache.shape[2], k_cache.shape[1], block_table.shape[1], d,
        int(window_left), int(num_splits), float(softmax_scale),
    )  # fmt: skip
    if rc != 0:
        raise MemoryError("oracle_paged_decode workspace allocation failed")
    return out


def native_paged_decode_partials(q, k_cache, v_cache, block_table, cache_seqlens, window_left, num_splits, softmax_scale):
    """The split kernel's ``(m, l, acc)`` partials, shapes ``(B*Hq, S)``, ``(B*Hq, S)``, ``(B*Hq, S, D)``."""
    b, hq, d = q.shape
    rows = b * hq
    sm = torch.empty(rows, num_splits)
    sl = torch.empty(rows, num_splits)
    sa = torch.empty(rows, num_splits, d)
    load().oracle_paged_decode_split(
        _fp(q), _fp(k_cache), _fp(v_cache), _ip(block_table), _ip(cache_seqlens), _fp(sm), _fp(sl), _fp(sa),
        b, hq, k_cache.shape[2], k_cache.shape[1], block_table.shape[1], d,
        int(window_left), int(num_splits), float(softmax_scale),
    )  # fmt: skip
    return sm, sl, sa


def native_reduce(sm, sl, sa):
    rows, splits, d = sa.shape
    out = torch.empty(rows, d)
    load().oracle_paged_decode_reduce(_fp(sm), _fp(sl), _fp(sa), _fp(out), rows, d, splits)
    return out


def native_varlen(q, k, v, cu_seqlens, window_left, softmax_scale):
    t, hq, d = q.shape
    out = torch.empty_like(q)
    load().oracle_varlen_forward(
        _fp(q), _fp(k), _fp(v), _fp(out), _ip(cu_seqlens), t, cu_seqlens.numel() - 1, hq, k.shape[1], d,
        int(window_left), float(softmax_scale),
    )  # fmt: skip
    return out
