"""Every unit of the matrix-core decode kernel's work list, walked on the CPU through the kernel's own item and cursor
functions (``areno_amd/csrc/decode_items.hpp`` compiled by g++ into ``tests/native/decode_walk.cpp``) with accessors
that check each index before use: item-table and prefix-sum indices, block-table columns, cached positions, partial
slots, and that the units read every cached token exactly once, in tile steps of 32 and of 64 tokens.  Workloads: the benchmark configurations at full size and the
shapes of the GPU parity tests that exercise prefix groups (32 / 8 heads x 8 samples, 400 groups of 3, overstated and
zero shared lengths), windows, empty rows and the largest batch."""

import ctypes
import os
import subprocess
import tempfile

import pytest
import torch

from areno_amd import workloads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def walker():
    out = os.path.join(tempfile.mkdtemp(prefix="decode_walk_"), "libdecode_walk.so")
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", out,
                    os.path.join(ROOT, "tests", "native", "decode_walk.cpp")], check=True)  # fmt: skip
    lib = ctypes.CDLL(out)
    lib.decode_walk.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p] + [ctypes.c_int] * 9 + [
        ctypes.POINTER(ctypes.c_longlong)] * 3 + [ctypes.c_char_p, ctypes.c_int]  # fmt: skip

    def walk(lengths, *, q_per_kv, units, shared=None, group_rows=1, window_left=-1, append_in_merge=1, tile_tokens=32,
             block_size=16, max_blocks=None, switch_quanta=3):  # fmt: skip
        lens = torch.as_tensor(lengths, dtype=torch.int32).contiguous()
        sh = None if shared is None else torch.as_tensor(shared, dtype=torch.int32).contiguous()
        if max_blocks is None:
            max_blocks = int(lens.max()) // block_size + 1
        quanta, partials, steps = ctypes.c_longlong(0), ctypes.c_longlong(0), ctypes.c_longlong(0)
        msg = ctypes.create_string_buffer(256)
        rc = lib.decode_walk(lens.data_ptr(), lens.numel(), None if sh is None else sh.data_ptr(), group_rows, q_per_kv,
                             window_left, append_in_merge, switch_quanta, units, tile_tokens, block_size, max_blocks,
                             ctypes.byref(quanta), ctypes.byref(partials), ctypes.byref(steps), msg, 256)  # fmt: skip
        assert rc == 0, msg.value.decode()
        return quanta.value, partials.value, steps.value

    return walk


def _expected_quanta(lengths, append_in_merge, window_left=-1):
    total = 0
    for n in [int(x) for x in lengths]:
        lo = 0 if window_left < 0 else max(0, n - window_left)
        total += max(0, -(-(n + 1 - append_in_merge - lo) // 16))
    return total


@pytest.mark.parametrize("append_in_merge", [0, 1])
@pytest.mark.parametrize("tile_tokens", [32, 64])
def test_cfg1_cfg2_units(walker, append_in_merge, tile_tokens):
    g = workloads._gen(1002 + 1)
    lengths = workloads._randint(g, 512, 4096, 64)
    quanta, partials, steps = walker(lengths, q_per_kv=7, units=256, append_in_merge=append_in_merge, tile_tokens=tile_tokens)
    assert quanta == _expected_quanta(lengths, append_in_merge)
    assert 256 <= partials <= 256 + 64
    # a unit's steps: its quanta in whole tiles, one more per segment border
    per_tile = tile_tokens // 16
    assert steps <= quanta // per_tile + 256 + 64 + 64


@pytest.mark.parametrize("append_in_merge", [0, 1])
def test_cfg3_full_size_with_and_without_groups(walker, append_in_merge):
    prefix, lengths = workloads.cfg3_lengths()
    shared = (prefix // 16) * 16
    plain, _, _ = walker(lengths, q_per_kv=4, units=512, append_in_merge=append_in_merge)
    grouped, _, _ = walker(lengths, q_per_kv=4, units=512, shared=shared, group_rows=8, append_in_merge=append_in_merge)
    assert plain == _expected_quanta(lengths, append_in_merge)
    # a prompt's shared tokens (cut to whole 32-token tiles) are read once per sub-group of 4 rows instead of once per row
    saved = sum(int(s) // 32 * 2 * (8 - 2) for s in shared)
    assert grouped == plain - saved


@pytest.mark.parametrize("hq,hkv,samples", [(32, 8, 8), (28, 4, 4), (8, 2, 3), (8, 8, 5)])
@pytest.mark.parametrize("units", [512, 1024, 2048])
def test_reduced_rollouts_of_the_gpu_tests(walker, hq, hkv, samples, units):
    prefix, lengths = workloads.cfg3_lengths(77, 6, samples, 8, 700, 120.0, 1.0, 900)
    shared = (prefix // 16) * 16
    walker(lengths, q_per_kv=hq // hkv, units=units, shared=shared, group_rows=samples)
    walker(lengths, q_per_kv=hq // hkv, units=units, shared=shared, group_rows=samples, append_in_merge=0, tile_tokens=32)


def test_groups_of_three_at_the_largest_launch(walker):
    prefix, lengths = workloads.cfg3_lengths(83, 400, 3, 40, 120, 30.0, 1.0, 100)
    shared = (prefix // 16) * 16
    # 1200 rows run as launches of 1023 and 177 rows (whole groups)
    for lo, hi in ((0, 1023), (1023, 1200)):
        walker(lengths[lo:hi], q_per_kv=4, units=2048, shared=shared[lo // 3 : hi // 3], group_rows=3)


def test_overstated_and_zero_shared_lengths(walker):
    prefix, lengths = workloads.cfg3_lengths(78, 3, 4, 64, 200, 50.0, 1.0, 300)
    shared = (prefix // 16) * 16
    shared[1] = 0
    walker(lengths, q_per_kv=4, units=1024, shared=shared, group_rows=4)
    walker(lengths, q_per_kv=4, units=1024, shared=shared * 0 + 100000, group_rows=4)  # clipped to the shortest member
    walker(lengths, q_per_kv=4, units=1024, shared=shared * 0 - 5, group_rows=4)  # negative claims share nothing


@pytest.mark.parametrize("window_left", [-1, 0, 40, 5000])
@pytest.mark.parametrize("append_in_merge", [0, 1])
@pytest.mark.parametrize("tile_tokens,switch_quanta", [(32, 3), (64, 3), (32, 0), (32, 1), (32, 7)])
def test_windows_empty_rows_and_page_borders(walker, window_left, append_in_merge, tile_tokens, switch_quanta):
    lengths = [0, 15, 16, 17, 31, 32, 33, 300, 0, 1, 4095, 0]
    kw = dict(window_left=window_left, append_in_merge=append_in_merge, tile_tokens=tile_tokens, switch_quanta=switch_quanta)
    quanta, _, _ = walker(lengths, q_per_kv=4, units=2048, **kw)
    assert quanta == _expected_quanta(lengths, append_in_merge, window_left)
    walker(lengths, q_per_kv=1, units=512, block_size=48, **kw)
    walker(lengths, q_per_kv=1, units=3, **kw)
    walker(lengths, q_per_kv=1, units=40, **kw)  # units of a few positions: some hold nothing but switch positions


def test_rows_at_the_end_of_their_block_table(walker):
    """A row whose next position has no column left (length = max_blocks * block_size): with the append folded into the
    merge launch the streaming waves read columns below max_blocks only."""
    walker([64, 32, 64], q_per_kv=4, units=64, block_size=16, max_blocks=4, append_in_merge=1)
    with pytest.raises(AssertionError, match="columns"):
        walker([64, 32, 64], q_per_kv=4, units=64, block_size=16, max_blocks=4, append_in_merge=0)


@pytest.mark.parametrize("lengths", [[800], [15], [4096], [40, 0, 7, 130], [1]])
@pytest.mark.parametrize("switch_quanta", [1, 3])
def test_launches_with_fewer_cost_positions_than_units(walker, lengths, switch_quanta):
    """A tiny batch has fewer cost positions than the launch has units: the first units take one position each and the
    others none, so a row's units are neighbours (the merge reads one partial per unit of the row's range)."""
    quanta, partials, _ = walker(lengths, q_per_kv=7, units=256, switch_quanta=switch_quanta)
    assert quanta == _expected_quanta(lengths, 1)
    assert partials <= quanta  # at most one partial per unit that holds a quantum


def test_batches_of_empty_rows(walker):
    assert walker([0, 0, 0], q_per_kv=4, units=1024)[0] == 0
    assert walker([0, 0, 5, 0], q_per_kv=4, units=1024)[0] == 1


def test_full_item_list(walker):
    g = torch.Generator().manual_seed(5)
    lengths = torch.randint(0, 90, (1024,), generator=g)
    walker(lengths, q_per_kv=4, units=2048)
    walker(lengths, q_per_kv=4, units=512, shared=torch.full((512,), 64), group_rows=2)  # 1024 rows + 512 shared items
