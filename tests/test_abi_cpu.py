"""The C-ABI library loads without a GPU and exports every symbol include/areno_hip.h declares;
argument validation (which runs before any launch) behaves as documented."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "areno_hip.h")
LIB = os.path.join(ROOT, "areno_amd", "accel", "libareno_hip.so")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(areno_hip_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is not built: run `python setup.py build_ext --inplace`")
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for required in ("areno_hip_cache_write", "areno_hip_cache_write_decode", "areno_hip_paged_decode",
                     "areno_hip_paged_decode_workspace_bytes", "areno_hip_paged_decode_grouped",
                     "areno_hip_paged_decode_grouped_workspace_bytes", "areno_hip_qk_norm_rope_cache_write",
                     "areno_hip_varlen_attention",
                     "areno_hip_paged_varlen_prefill", "areno_hip_prefill_workspace_bytes", "areno_hip_abi_version",
                     "areno_hip_block_tables_init", "areno_hip_block_tables_reserve",
                     "areno_hip_block_tables_ensure_decode", "areno_hip_block_tables_release",
                     "areno_hip_block_tables_gather", "areno_hip_block_tables_decode_step",
                     "areno_hip_block_tables_prefill_slots", "areno_hip_attention_backward", "areno_hip_attention_backward_typed", "areno_hip_probe_mfma_rate",
                     "areno_hip_attention_backward_workspace_bytes", "areno_hip_paged_decode_plan",
                     "areno_hip_paged_decode_plan_bytes", "areno_hip_paged_decode_planned", "areno_hip_rope_rows",
                     "areno_hip_rope_rows_bytes", "areno_hip_qk_norm_rope_cache_write_rows"):  # fmt: skip
        assert required in names


def test_library_exports_every_declared_symbol(lib):
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/areno_hip.h but not exported"


def test_version_status_strings_and_workspace_size(lib):
    assert lib.areno_hip_abi_version() == 1
    lib.areno_hip_status_string.restype = ctypes.c_char_p
    assert lib.areno_hip_status_string(0) == b"ok"
    assert b"workspace" in lib.areno_hip_status_string(-3)
    ws = lib.areno_hip_paged_decode_workspace_bytes
    ws.restype = ctypes.c_size_t
    ws.argtypes = [ctypes.c_int32] * 6
    # two layouts share the workspace: fixed chunks (B * Hq * chunks rows) and the balanced-piece layout
    # ((256 workgroups * 4 waves + B) * Hq rows, the dump row of the lanes that own no partial -- 16 columns of the widest
    # head and an (m, l) pair per lane -- plus the B + 1 prefix sums); the size is the larger of the two
    def pieces(b, hq, d):
        rows = ((1024 + b) * hq * (d + 2) + 16 * 512 + 2 * 64) * 4
        return (rows + 255) // 256 * 256 + (b + 1 + 63) // 64 * 64 * 4

    # B=64, Hq=28, D=128, bs=16, MB=257: 4112 tokens -> 17 chunks of 256
    assert ws(64, 28, 128, 16, 257, 8) == max(64 * 28 * 17 * 130 * 4, pieces(64, 28, 128))
    assert ws(4096, 28, 128, 16, 257, 8) == max(4096 * 28 * 17 * 130 * 4, pieces(4096, 28, 128))
    assert ws(0, 28, 128, 16, 257, 8) == 0 and ws(64, 28, 128, 16, 257, 0) == 0
    # long tables fold into at most 64 chunks per row
    assert ws(4096, 1, 128, 16, 4096, 8) == max(4096 * 64 * 130 * 4, pieces(4096, 1, 128))


def test_argument_validation_runs_before_any_launch(lib):
    class Cache(ctypes.Structure):
        _fields_ = [("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("k_scale", ctypes.c_void_p),
                    ("v_scale", ctypes.c_void_p), ("num_blocks", ctypes.c_int64), ("block_size", ctypes.c_int32),
                    ("kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("cache_dtype", ctypes.c_int32),
                    ("scale_dtype", ctypes.c_int32)]  # fmt: skip

    lib.areno_hip_last_error.restype = ctypes.c_char_p
    fn = lib.areno_hip_cache_write
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                   ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]  # fmt: skip
    assert fn(None, None, None, 2, 1, None, None, None) == -1
    cache = Cache(None, None, None, None, 4, 16, 2, 64, 2, 0)
    assert fn(ctypes.byref(cache), None, None, 2, 0, None, None, None) == -1  # NULL pools
    assert b"NULL" in lib.areno_hip_last_error()
    cache = Cache(0x1000, 0x1000, None, None, 4, 16, 2, 64, 3, 1)  # int8 cache without scales
    assert fn(ctypes.byref(cache), 0x1000, 0x1000, 2, 0, None, None, None) == -1
    assert b"k_scale" in lib.areno_hip_last_error()
    cache = Cache(0x1000, 0x1000, None, None, 4, 16, 2, 64, 2, 0)
    assert fn(ctypes.byref(cache), 0x1000, 0x1000, 1, 0, None, None, None) == -2  # f16 rows into a bf16 cache
    assert fn(ctypes.byref(cache), 0x1000, 0x1000, 2, 0, None, None, None) == 0  # zero tokens: nothing to do


def test_the_fused_front_step_refuses_sizes_past_its_32_bit_indexing(lib):
    """areno_hip_qk_norm_rope_cache_write indexes rows, elements and page rows with 32 bits; the launcher turns tables and
    pools past that down by name before anything is launched (fake pointers: nothing dereferences them).  Token counts
    past it run as several launches: tests/test_gpu_rope_write.py."""
    class Cache(ctypes.Structure):
        _fields_ = [("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("k_scale", ctypes.c_void_p),
                    ("v_scale", ctypes.c_void_p), ("num_blocks", ctypes.c_int64), ("block_size", ctypes.c_int32),
                    ("kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("cache_dtype", ctypes.c_int32),
                    ("scale_dtype", ctypes.c_int32)]  # fmt: skip

    lib.areno_hip_last_error.restype = ctypes.c_char_p
    fn = lib.areno_hip_qk_norm_rope_cache_write
    fn.restype = ctypes.c_int
    p, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
    fn.argtypes = [p, p, p, p, p, p, i32, i64, i32, i32, i32, p, p, p, i32, p, p, f32, p, p, p]
    fake = 0x1000
    bf16, unsupported = 2, -2

    def call(cache, tokens, q_heads, kv_heads, d, max_pos=4096):
        return fn(cache, fake, fake, fake, fake, fake, bf16, tokens, q_heads, kv_heads, d, fake, fake, fake, max_pos,
                  None, None, 1e-6, fake, fake, None)  # fmt: skip

    assert call(None, 16, 8, 2, 128, max_pos=1 << 24) == unsupported  # rotary table offsets
    assert b"32-bit" in lib.areno_hip_last_error()
    pool = Cache(fake, fake, None, None, 1 << 29, 16, 2, 128, bf16, 0)  # 2^33 page rows
    assert call(ctypes.byref(pool), 16, 8, 2, 128) == unsupported
    assert b"page rows" in lib.areno_hip_last_error()
    assert call(None, 0, 8, 2, 128) == 0  # nothing to do
