"""ctypes mirror of ``include/areno_hip.h``: calls ``libareno_hip.so`` with raw device pointers.

This is the binding a non-PyTorch host would write; the benchmark and the C-ABI tests use it to drive
single kernels (stage masks) without going through the torch extension.  Tensors are only used here to
obtain ``data_ptr()`` and shapes.
"""

from __future__ import annotations

import ctypes

import torch

from areno_amd.accel._extension import library_path

DT_F32, DT_F16, DT_BF16, DT_I8, DT_FP8_E4M3 = 0, 1, 2, 3, 4
STAGE_APPEND, STAGE_SPLIT, STAGE_REDUCE, STAGE_ALL = 1, 2, 4, 7
OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_LAUNCH = 0, -1, -2, -3, -4

_DTYPE_CODES = {
    torch.float32: DT_F32,
    torch.float16: DT_F16,
    torch.bfloat16: DT_BF16,
    torch.int8: DT_I8,
    torch.float8_e4m3fn: DT_FP8_E4M3,
}


class PagedCache(ctypes.Structure):
    """``struct areno_paged_cache``."""

    _fields_ = [
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("k_scale", ctypes.c_void_p),
        ("v_scale", ctypes.c_void_p),
        ("num_blocks", ctypes.c_int64),
        ("block_size", ctypes.c_int32),
        ("kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("cache_dtype", ctypes.c_int32),
        ("scale_dtype", ctypes.c_int32),
    ]


class DecodePlan(ctypes.Structure):
    """``struct areno_decode_plan``."""

    _fields_ = [("buffer", ctypes.c_void_p), ("buffer_bytes", ctypes.c_size_t)] + [
        (name, ctypes.c_int32)
        for name in ("batch", "q_heads", "kv_heads", "head_dim", "block_size", "max_blocks", "window_left", "cache_dtype",
                     "q_dtype", "with_update", "group_rows", "units", "items", "tile_tokens")
    ]  # fmt: skip


class BlockTables(ctypes.Structure):
    """``struct areno_block_tables``."""

    _fields_ = [
        ("table", ctypes.c_void_p),
        ("row_blocks", ctypes.c_void_p),
        ("free_ring", ctypes.c_void_p),
        ("state", ctypes.c_void_p),
        ("max_rows", ctypes.c_int32),
        ("max_blocks", ctypes.c_int32),
        ("num_blocks", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
    ]


PAD_LAST_BLOCK, PAD_SCRATCH_BLOCK = 0, 1

_LIB: ctypes.CDLL | None = None
_P, _I32, _I64, _F, _SZ = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        try:
            handle = ctypes.CDLL(library_path())
        except OSError as exc:
            raise RuntimeError(
                f"libareno_hip.so could not be loaded ({exc}); build it with `python setup.py build_ext --inplace`"
            ) from exc
        handle.areno_hip_last_error.restype = ctypes.c_char_p
        handle.areno_hip_status_string.restype = ctypes.c_char_p
        handle.areno_hip_paged_decode_workspace_bytes.restype = _SZ
        handle.areno_hip_paged_decode_workspace_bytes.argtypes = [_I32] * 6
        handle.areno_hip_cache_write.argtypes = [_P, _P, _P, _I32, _I64, _P, _P, _P]
        handle.areno_hip_cache_write_decode.argtypes = [_P, _P, _P, _I32, _I32, _P, _I32, _P, _P]
        decode_args = [_P, _P, _P, _P, _P, _I32, _I32, _I32, _P, _I32, _P, _I32, _I32, _F, _P, _SZ]
        handle.areno_hip_paged_decode.argtypes = decode_args + [_P]
        handle.areno_hip_paged_decode_stages.argtypes = decode_args + [_I32, _P]
        handle.areno_hip_paged_decode_static.argtypes = decode_args[:-2] + [_P]
        handle.areno_hip_paged_decode_static_capacity.restype = _SZ
        handle.areno_hip_paged_decode_static_capacity.argtypes = []
        handle.areno_hip_paged_decode_grouped.argtypes = decode_args[:-2] + [_I32, _P, _P, _SZ, _I32, _P]
        handle.areno_hip_paged_decode_grouped_workspace_bytes.restype = _SZ
        handle.areno_hip_paged_decode_grouped_workspace_bytes.argtypes = [_I32] * 8
        handle.areno_hip_paged_decode_plan_bytes.restype = _SZ
        handle.areno_hip_paged_decode_plan_bytes.argtypes = [_I32]
        handle.areno_hip_paged_decode_plan.argtypes = [_P, _P, _SZ, _P, _I32, _I32, _I32, _P, _I32, _P, _I32, _I32, _I32, _P, _P]
        handle.areno_hip_paged_decode_planned.argtypes = decode_args[:-2] + [_I32, _P, _P, _P, _SZ, _I32, _P]
        handle.areno_hip_varlen_attention.argtypes = [_P, _P, _P, _P, _I32, _I64, _I32, _I32, _I32, _P, _I32, _I32, _F, _P, _SZ, _P]  # fmt: skip
        handle.areno_hip_paged_varlen_prefill.argtypes = [_P, _P, _P, _I32, _I64, _I32, _I32, _P, _I32, _P, _P, _I32, _F, _P, _SZ, _P]  # fmt: skip
        handle.areno_hip_prefill_workspace_bytes.restype = _SZ
        handle.areno_hip_prefill_workspace_bytes.argtypes = [_I32, _I32]
        handle.areno_hip_probe_stream_read.argtypes = [_P, _P, _P, _I64, _I32, _I32, _P, _P]
        handle.areno_hip_probe_mfma_rate.restype = _I64
        handle.areno_hip_probe_mfma_rate.argtypes = [_I32, _I32, _P, _P]
        handle.areno_hip_block_tables_init.argtypes = [_P, _P]
        handle.areno_hip_block_tables_reserve.argtypes = [_P, _P, _P, _I32, _P]
        handle.areno_hip_block_tables_ensure_decode.argtypes = [_P, _P, _P, _I32, _P]
        handle.areno_hip_block_tables_release.argtypes = [_P, _P, _I32, _P]
        handle.areno_hip_block_tables_gather.argtypes = [_P, _P, _I32, _I32, _P, _P]
        handle.areno_hip_block_tables_decode_step.argtypes = [_P, _P, _P, _I32, _I32, _P, _P]
        handle.areno_hip_block_tables_prefill_slots.argtypes = [_P, _P, _P, _P, _I32, _I64, _P, _P, _P, _P]
        _LIB = handle
    return _LIB


def check(status: int, op: str) -> None:
    if status != 0:
        handle = lib()
        raise RuntimeError(
            f"{op} failed: {handle.areno_hip_status_string(status).decode()} ({handle.areno_hip_last_error().decode()})"
        )


def dtype_code(t: torch.Tensor) -> int:
    return _DTYPE_CODES[t.dtype]


def describe_cache(k_cache, v_cache, k_scale=None, v_scale=None) -> PagedCache:
    nb, bs, hkv, d = k_cache.shape
    return PagedCache(
        k_cache.data_ptr(), v_cache.data_ptr(),
        None if k_scale is None else k_scale.data_ptr(), None if v_scale is None else v_scale.data_ptr(),
        nb, bs, hkv, d, dtype_code(k_cache),
        DT_F32 if k_scale is None else dtype_code(k_scale),
    )  # fmt: skip


def current_stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def decode_workspace_bytes(batch, q_heads, head_dim, block_size, max_blocks, num_splits=8) -> int:
    return int(lib().areno_hip_paged_decode_workspace_bytes(batch, q_heads, head_dim, block_size, max_blocks, num_splits))


def decode_grouped_workspace_bytes(batch, q_heads, kv_heads, head_dim, block_size, max_blocks, group_rows,
                                   num_splits=8) -> int:  # fmt: skip
    return int(lib().areno_hip_paged_decode_grouped_workspace_bytes(batch, q_heads, kv_heads, head_dim, block_size,
                                                                    max_blocks, num_splits, group_rows))  # fmt: skip


def decode_plan_bytes(batch: int) -> int:
    return int(lib().areno_hip_paged_decode_plan_bytes(int(batch)))


def paged_decode_plan(cache: PagedCache, q_dtype: torch.dtype, q_heads: int, block_table, cache_seqlens, buffer, *,
                      window_left=-1, with_update=True, group_rows=None, shared_lens=None, stream=None) -> DecodePlan:  # fmt: skip
    """``areno_hip_paged_decode_plan`` on raw pointers: fills ``buffer`` (a uint8 device tensor of at least
    ``decode_plan_bytes(batch)`` bytes, which must outlive the plan) and returns the host-side description."""
    plan = DecodePlan()
    check(lib().areno_hip_paged_decode_plan(
        ctypes.byref(plan), buffer.data_ptr(), buffer.numel(), ctypes.byref(cache), _DTYPE_CODES[q_dtype],
        block_table.shape[0], int(q_heads), block_table.data_ptr(), block_table.shape[1], cache_seqlens.data_ptr(),
        int(window_left), 1 if with_update else 0, 0 if shared_lens is None else int(group_rows),
        None if shared_lens is None else shared_lens.data_ptr(), current_stream_ptr() if stream is None else stream,
    ), "areno_hip_paged_decode_plan")  # fmt: skip
    return plan


def paged_decode(cache: PagedCache, q, k_update, v_update, out, block_table, cache_seqlens, workspace, *,
                 window_left=-1, num_splits=8, softmax_scale=None, stages=STAGE_ALL, stream=None,
                 group_rows=None, shared_lens=None, plan: DecodePlan | None = None) -> None:  # fmt: skip
    """``areno_hip_paged_decode_stages`` (``_grouped`` when ``shared_lens`` is given, ``_planned`` with a plan) on raw
    pointers; ``workspace`` is a uint8 device tensor."""
    scale = float(softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5)
    if plan is not None:
        status = lib().areno_hip_paged_decode_planned(
            ctypes.byref(cache), q.data_ptr(), None if k_update is None else k_update.data_ptr(),
            None if v_update is None else v_update.data_ptr(), out.data_ptr(), dtype_code(q), q.shape[0], q.shape[1],
            block_table.data_ptr(), block_table.shape[1], cache_seqlens.data_ptr(), int(window_left), int(num_splits),
            scale, 0 if shared_lens is None else int(group_rows), None if shared_lens is None else shared_lens.data_ptr(),
            ctypes.byref(plan), workspace.data_ptr(), workspace.numel(), int(stages),
            current_stream_ptr() if stream is None else stream,
        )  # fmt: skip
        check(status, "areno_hip_paged_decode_planned")
        return
    if shared_lens is not None:
        status = lib().areno_hip_paged_decode_grouped(
            ctypes.byref(cache), q.data_ptr(), None if k_update is None else k_update.data_ptr(),
            None if v_update is None else v_update.data_ptr(), out.data_ptr(), dtype_code(q), q.shape[0], q.shape[1],
            block_table.data_ptr(), block_table.shape[1], cache_seqlens.data_ptr(), int(window_left), int(num_splits),
            scale, int(group_rows), shared_lens.data_ptr(), workspace.data_ptr(), workspace.numel(), int(stages),
            current_stream_ptr() if stream is None else stream,
        )  # fmt: skip
        check(status, "areno_hip_paged_decode_grouped")
        return
    status = lib().areno_hip_paged_decode_stages(
        ctypes.byref(cache), q.data_ptr(), None if k_update is None else k_update.data_ptr(),
        None if v_update is None else v_update.data_ptr(), out.data_ptr(), dtype_code(q), q.shape[0], q.shape[1],
        block_table.data_ptr(), block_table.shape[1], cache_seqlens.data_ptr(), int(window_left), int(num_splits),
        scale, workspace.data_ptr(), workspace.numel(), int(stages),
        current_stream_ptr() if stream is None else stream,
    )  # fmt: skip
    check(status, "areno_hip_paged_decode")


def paged_decode_static(cache: PagedCache, q, k_update, v_update, out, block_table, cache_seqlens, *, window_left=-1,
                        num_splits=8, softmax_scale=None, stream=None) -> int:  # fmt: skip
    """``areno_hip_paged_decode_static`` (the decode op on the library's built-in scratch buffer) on raw pointers;
    returns the status code."""
    scale = float(softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5)
    return int(lib().areno_hip_paged_decode_static(
        ctypes.byref(cache), q.data_ptr(), None if k_update is None else k_update.data_ptr(),
        None if v_update is None else v_update.data_ptr(), out.data_ptr(), dtype_code(q), q.shape[0], q.shape[1],
        block_table.data_ptr(), block_table.shape[1], cache_seqlens.data_ptr(), int(window_left), int(num_splits),
        scale, current_stream_ptr() if stream is None else stream,
    ))  # fmt: skip


def probe_stream_read(pool_a, pool_b, page_bytes: int, sink, page_ids=None, stream=None, prefetch_ids=False) -> int:
    """``areno_hip_probe_stream_read`` over two device tensors (K and V pool) cut into runs of ``page_bytes``: all of
    them, in order, or the runs an int32 tensor of ids names (``prefetch_ids``: each wave fetches its next id a run
    ahead).  Returns the bytes one call reads."""
    pages = (pool_a.numel() * pool_a.element_size()) // page_bytes if page_ids is None else page_ids.numel()
    check(lib().areno_hip_probe_stream_read(pool_a.data_ptr(), None if pool_b is None else pool_b.data_ptr(),
                                            None if page_ids is None else page_ids.data_ptr(), pages, page_bytes,
                                            1 if prefetch_ids else 0, sink.data_ptr(),
                                            current_stream_ptr() if stream is None else stream),
          "areno_hip_probe_stream_read")  # fmt: skip
    return pages * page_bytes * (1 if pool_b is None else 2)


def probe_mfma_rate(shape: int, iters: int, sink, stream=None) -> int:
    """``areno_hip_probe_mfma_rate``: one launch of independent matrix products of a shape (0: 16 x 16 x 32 bf16,
    1: 32 x 32 x 16 bf16, 2 / 3: the same in f16); returns the launch's floating-point operations."""
    flops = int(lib().areno_hip_probe_mfma_rate(int(shape), int(iters), sink.data_ptr(),
                                                current_stream_ptr() if stream is None else stream))  # fmt: skip
    if flops < 0:
        check(-1, "areno_hip_probe_mfma_rate")
    return flops


def prefill_workspace_bytes(kv_heads: int, head_dim: int) -> int:
    return int(lib().areno_hip_prefill_workspace_bytes(int(kv_heads), int(head_dim)))


def paged_varlen_prefill(cache: PagedCache, q, out, block_table, cu_seqlens_q, context_lens, workspace, *,
                         window_left=-1, softmax_scale=None, workspace_bytes=None, stream=None) -> int:  # fmt: skip
    """``areno_hip_paged_varlen_prefill`` on raw pointers; returns the status code instead of raising, so a caller
    can probe error paths (``check`` turns it into an exception)."""
    scale = float(softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5)
    return int(lib().areno_hip_paged_varlen_prefill(
        ctypes.byref(cache), q.data_ptr(), out.data_ptr(), dtype_code(q), q.shape[0], q.shape[1],
        context_lens.shape[0], block_table.data_ptr(), block_table.shape[1], cu_seqlens_q.data_ptr(),
        context_lens.data_ptr(), int(window_left), scale, workspace.data_ptr(),
        workspace.numel() if workspace_bytes is None else int(workspace_bytes),
        current_stream_ptr() if stream is None else stream,
    ))  # fmt: skip


def describe_block_tables(table, row_blocks, free_ring, state, block_size: int) -> BlockTables:
    """Descriptor over four int32 device tensors: table [rows, max_blocks], row_blocks [rows], free_ring [pages],
    state [4]."""
    return BlockTables(table.data_ptr(), row_blocks.data_ptr(), free_ring.data_ptr(), state.data_ptr(),
                       table.shape[0], table.shape[1], free_ring.shape[0], block_size)  # fmt: skip


def block_tables_init(bt: BlockTables) -> int:
    return lib().areno_hip_block_tables_init(ctypes.byref(bt), current_stream_ptr())


def block_tables_reserve(bt: BlockTables, rows, token_counts) -> int:
    return lib().areno_hip_block_tables_reserve(ctypes.byref(bt), rows.data_ptr(), token_counts.data_ptr(),
                                                rows.numel(), current_stream_ptr())  # fmt: skip


def block_tables_ensure_decode(bt: BlockTables, rows, next_positions) -> int:
    return lib().areno_hip_block_tables_ensure_decode(ctypes.byref(bt), rows.data_ptr(), next_positions.data_ptr(),
                                                      rows.numel(), current_stream_ptr())  # fmt: skip


def block_tables_release(bt: BlockTables, rows) -> int:
    return lib().areno_hip_block_tables_release(ctypes.byref(bt), rows.data_ptr(), rows.numel(), current_stream_ptr())


def block_tables_gather(bt: BlockTables, rows, pad_mode: int, out_table) -> int:
    return lib().areno_hip_block_tables_gather(ctypes.byref(bt), rows.data_ptr(), rows.numel(), pad_mode,
                                               out_table.data_ptr(), current_stream_ptr())  # fmt: skip


def block_tables_decode_step(bt: BlockTables, rows, next_positions, pad_mode: int, out_table) -> int:
    return lib().areno_hip_block_tables_decode_step(ctypes.byref(bt), rows.data_ptr(), next_positions.data_ptr(),
                                                    rows.numel(), pad_mode, out_table.data_ptr(),
                                                    current_stream_ptr())  # fmt: skip


def block_tables_prefill_slots(bt: BlockTables, rows, cursors, cu_seqlens, tokens: int, out_ids, out_offsets,
                               out_positions=None) -> int:  # fmt: skip
    return lib().areno_hip_block_tables_prefill_slots(
        ctypes.byref(bt), rows.data_ptr(), cursors.data_ptr(), cu_seqlens.data_ptr(), rows.numel(), tokens,
        out_ids.data_ptr(), out_offsets.data_ptr(), None if out_positions is None else out_positions.data_ptr(),
        current_stream_ptr(),
    )
