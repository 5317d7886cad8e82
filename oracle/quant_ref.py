"""Closed-form KV quantizers of this build (CPU restatement).

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

The reference has no quantized KV cache; the only in-tree precedent for the
int8 recipe is its 8-bit optimizer (``areno/engine/optim/adamw_8bit.py:263-276``:
``scale = absmax / 127``, round, clamp).  Both quantizers work per
``(token, kv_head)`` row of ``D`` elements:

int8    a = max|x| (fp32); s = fp16_rne(min(a / 127, 65504)); s == 0 -> s = 1;
        code = clamp(rne(x / float(s)), -127, 127); x^ = code * float(s)
fp8     a = max|x| (fp32); s = a / 448 (fp32); s == 0 -> s = 1;
        code = e4m3fn_rne(clamp(x / s, -448, 448));   x^ = float(code) * s

Divisions are IEEE fp32 divisions, rounding is round-half-to-even.
"""

from __future__ import annotations

import numpy as np
import torch

INT8_QMAX = 127.0
FP8_E4M3_MAX = 448.0
FP16_MAX = 65504.0


def quantize_int8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``x (..., D)`` -> ``(codes int8 (..., D), scales fp16 (...))``."""
    xf = x.float()
    absmax = xf.abs().amax(dim=-1)
    s32 = torch.clamp(absmax / INT8_QMAX, max=FP16_MAX)
    s16 = s32.to(torch.float16)
    s16 = torch.where(s16 == 0, torch.ones_like(s16), s16)
    codes = torch.clamp(torch.round(xf / s16.float().unsqueeze(-1)), -INT8_QMAX, INT8_QMAX)
    return codes.to(torch.int8), s16


def quantize_fp8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``x (..., D)`` -> ``(codes float8_e4m3fn (..., D), scales fp32 (...))``."""
    xf = x.float()
    absmax = xf.abs().amax(dim=-1)
    s32 = absmax / FP8_E4M3_MAX
    s32 = torch.where(s32 == 0, torch.ones_like(s32), s32)
    y = torch.clamp(xf / s32.unsqueeze(-1), -FP8_E4M3_MAX, FP8_E4M3_MAX)
    return y.to(torch.float8_e4m3fn), s32


def quantize(x: torch.Tensor, cache_dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    if cache_dtype == torch.int8:
        return quantize_int8(x)
    if cache_dtype == torch.float8_e4m3fn:
        return quantize_fp8(x)
    raise ValueError(f"not a quantized cache dtype: {cache_dtype}")


def dequantize(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """fp32 ``codes * scales[..., None]`` (exact: one fp32 multiply per element)."""
    return codes.float() * scales.float().unsqueeze(-1)


def e4m3fn_decode_table() -> np.ndarray:
    """All 256 OCP FP8 E4M3 ("fn": no infinities, 0x7f/0xff are NaN) values, from the bit layout.

    sign(1) exponent(4, bias 7) mantissa(3); exponent 0 is subnormal: ``m/8 * 2**-6``.
    """
    out = np.empty(256, dtype=np.float64)
    for b in range(256):
        sign = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 0x7
        if e == 0xF and m == 0x7:
            out[b] = np.nan
        elif e == 0:
            out[b] = sign * (m / 8.0) * 2.0**-6
        else:
            out[b] = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


def e4m3fn_encode_bruteforce(y: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even onto the finite E4M3 grid by exhaustive search (|y| <= 448)."""
    table = e4m3fn_decode_table()
    finite = np.array([b for b in range(256) if not np.isnan(table[b]) and not (b == 0x80)], dtype=np.int64)
    vals = table[finite]
    order = np.argsort(vals, kind="stable")
    vals, finite = vals[order], finite[order]
    y = np.asarray(y, dtype=np.float64)
    hi = np.clip(np.searchsorted(vals, y, side="left"), 0, len(vals) - 1)
    lo = np.clip(hi - 1, 0, len(vals) - 1)
    d_lo, d_hi = np.abs(y - vals[lo]), np.abs(vals[hi] - y)
    pick_hi = d_hi < d_lo
    tie = d_hi == d_lo
    even_hi = (finite[hi] & 1) == 0
    idx = np.where(pick_hi | (tie & even_hi), hi, lo)
    codes = finite[idx].astype(np.uint8)
    # signed zero: tiny negatives round to -0 (0x80), like an IEEE-style cast
    codes = np.where((vals[idx] == 0) & np.signbit(y), np.uint8(0x80), codes)
    return codes


def ref_quantized_cache_write(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_scale: torch.Tensor,
    v_scale: torch.Tensor,
    cache_block_ids: torch.Tensor,
    cache_block_offsets: torch.Tensor,
) -> None:
    """Quantize-and-scatter: codes to ``cache[ids, offs]``, scales to ``scale[ids, offs]``.

    Addressing as ``_store_prefill_cache`` (``attention_backend/infer.py:245-263``).
    """
    ids, offs = cache_block_ids.long(), cache_block_offsets.long()
    kc, ks = quantize(key, k_cache.dtype)
    vc, vs = quantize(value, v_cache.dtype)
    # index_put_ on float8 is not implemented on every torch build: scatter the raw bytes.
    k_cache.view(torch.uint8).index_put_((ids, offs), kc.view(torch.uint8))
    v_cache.view(torch.uint8).index_put_((ids, offs), vc.view(torch.uint8))
    k_scale.index_put_((ids, offs), ks.to(k_scale.dtype))
    v_scale.index_put_((ids, offs), vs.to(v_scale.dtype))


def decode_addresses(block_table: torch.Tensor, cache_seqlens: torch.Tensor, block_size: int):
    """``(block id, slot)`` of the token each decode row appends (``attention.cu:545-549``)."""
    pos = cache_seqlens.long()
    cols = torch.div(pos, block_size, rounding_mode="floor")
    ids = block_table.long()[torch.arange(block_table.shape[0]), cols]
    return ids, pos % block_size
