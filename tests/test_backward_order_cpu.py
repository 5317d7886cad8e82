"""The order in which the matrix-core backward kernels' workgroups take the blocks of packed rows
(``areno_amd/csrc/backward_order.hpp`` compiled by g++ into ``tests/native/backward_order.cpp``): a permutation for
every number of blocks and sequences, and by cost when the sequences are equally long."""

import ctypes
import os
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_block_order_is_a_permutation_and_goes_by_cost():
    out = os.path.join(tempfile.mkdtemp(prefix="backward_order_"), "libbackward_order.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", out,
                    os.path.join(ROOT, "tests", "native", "backward_order.cpp")], check=True)  # fmt: skip
    lib = ctypes.CDLL(out)
    lib.backward_order_check.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_longlong), ctypes.c_char_p, ctypes.c_int]
    cases = ctypes.c_longlong(0)
    msg = ctypes.create_string_buffer(256)
    rc = lib.backward_order_check(200, 210, ctypes.byref(cases), msg, 256)
    assert rc == 0, msg.value.decode()
    assert cases.value == 200 * 211 * 2
