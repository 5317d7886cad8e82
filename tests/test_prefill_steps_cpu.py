"""The prefill kernel's step geometry on the CPU (``areno_amd/csrc/prefill_steps.hpp`` compiled by g++ into
``tests/native/prefill_steps.cpp``): the closed form for the tile steps in front of a query block and the bisection
that finds the block of a step against a walk over the blocks, exhaustively over small shapes (every block size the
kernel uses, windows around the tile size, contexts and lengths around tile and block borders) and on large and
random ones."""

import ctypes
import os
import random
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# rows per workgroup (64, 128, 256) over the q heads folded into a block's rows (1 .. 16): powers of two, and what
# groups of 3, 5, 6, 7, 9 .. 15 heads give
BLOCK_TOKENS = [4, 8, 16, 32, 64, 128, 256, 85, 51, 42, 36, 28, 25, 23, 21, 19, 18, 17, 12, 10, 9, 7, 5]


@pytest.fixture(scope="module")
def lib():
    out = os.path.join(tempfile.mkdtemp(prefix="prefill_steps_"), "libprefill_steps.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", out,
                    os.path.join(ROOT, "tests", "native", "prefill_steps.cpp")], check=True)  # fmt: skip
    lib = ctypes.CDLL(out)
    lib.prefill_steps_check.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_longlong), ctypes.c_char_p, ctypes.c_int]
    lib.prefill_steps_check_grid.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                                             ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                                             ctypes.POINTER(ctypes.c_longlong), ctypes.c_char_p, ctypes.c_int]  # fmt: skip
    return lib


def test_closed_forms_on_every_small_shape(lib):
    windows = [-1, 0, 1, 3, 15, 16, 31, 32, 33, 63, 64, 65, 100, 257]
    tqs = (ctypes.c_int * len(BLOCK_TOKENS))(*BLOCK_TOKENS)
    ws = (ctypes.c_int * len(windows))(*windows)
    shapes = ctypes.c_longlong(0)
    msg = ctypes.create_string_buffer(256)
    rc = lib.prefill_steps_check_grid(150, 100, tqs, len(BLOCK_TOKENS), ws, len(windows), ctypes.byref(shapes), msg, 256)
    assert rc == 0, msg.value.decode()
    assert shapes.value == len(BLOCK_TOKENS) * len(windows) * 101 * 151


def test_closed_forms_on_large_and_random_shapes(lib):
    rng = random.Random(5)
    msg = ctypes.create_string_buffer(256)
    steps = ctypes.c_longlong(0)
    cases = [(4096, 0, 64, -1), (8192, 0, 16, -1), (1, 1 << 20, 4, -1), (100000, 900000, 4, 5000), (65536, 12345, 256, 1),
             (512, 16384, 64, -1), (300000, 0, 8, 31), (1 << 20, 1 << 20, 256, 1 << 19), (100000, 77, 36, -1),
             (4096, 0, 36, 100), (250000, 123456, 9, 4000), (65536, 31, 85, 33)]  # fmt: skip
    for _ in range(300):
        cases.append((rng.randrange(0, 20000), rng.randrange(0, 100000), rng.choice(BLOCK_TOKENS),
                      rng.choice([-1, -1, rng.randrange(0, 50000)])))  # fmt: skip
    for n_new, ctx, tq, window in cases:
        rc = lib.prefill_steps_check(n_new, ctx, tq, window, 0, ctypes.byref(steps), msg, 256)
        assert rc == 0, msg.value.decode()
    # a known total: 4 096 new tokens without context in blocks of 64 see 2 j + 2 tiles each
    lib.prefill_steps_check(4096, 0, 64, -1, 0, ctypes.byref(steps), msg, 256)
    assert steps.value == sum(2 * j + 2 for j in range(64))
