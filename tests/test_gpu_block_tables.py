"""Device-resident page bookkeeping vs the host restatement of the reference's lists (oracle/block_table_ref.py):
after every call the device state -- free list in order, each row's pages in order, status word -- must equal the
oracle's, i.e. a row holds exactly the page ids the reference's scheduler would have given it
(areno/engine/data/rollout_state.py:128-151,212-225,282-285, areno/engine/inference.py:573-580,651-658).  Integer
work: the bar is equality."""

import random

import pytest
import torch

from areno_amd.accel import cabi
from areno_amd.engine import DeviceBlockTables
from oracle.block_table_ref import BAD_ROW, EXHAUSTED, OK, ROW_FULL, RefBlockTables
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _same_state(dev: DeviceBlockTables, ref: RefBlockTables):
    assert dev.free_list() == ref.free_list()
    counts = dev.row_blocks.cpu().tolist()
    table = dev.table.cpu().tolist()
    for row in range(ref.max_rows):
        assert table[row][: counts[row]] == ref.row_pages(row), f"row {row}"
    assert dev.status() == (ref.status, ref.first_fail)


def test_values_of_the_reference_scheduler_test():
    # tests/test_inference_scheduler_cpu.py:135-156 in the reference
    dev = DeviceBlockTables(2, 1, 32, 4, DEV)
    dev.reserve([0], [2])
    assert dev.row_pages(0) == [0] and dev.free_list() == [1]
    dev.ensure_decode(torch.tensor([0], device=DEV), torch.tensor([4], dtype=torch.int32, device=DEV))
    assert dev.row_pages(0) == [0, 1] and dev.free_list() == [] and dev.status() == (OK, -1)
    dev.check()


@pytest.mark.parametrize("seed,num_blocks,max_rows,max_blocks,bs", [
    (1, 40, 12, 6, 4), (2, 700, 300, 9, 16), (3, 64, 64, 64, 1), (4, 5000, 1500, 8, 16)])  # fmt: skip
def test_random_traffic_matches_the_host_lists(seed, num_blocks, max_rows, max_blocks, bs):
    """Admissions, decode steps and releases in random order, tight enough that the pool runs dry now and then;
    more than 1024 rows exercises the second pass of the one-workgroup kernels."""
    rng = random.Random(seed)
    dev = DeviceBlockTables(num_blocks, max_rows, max_blocks, bs, DEV)
    ref = RefBlockTables(num_blocks, max_rows, max_blocks, bs)
    lengths: dict[int, int] = {}
    for step in range(60):
        op = rng.random()
        if op < 0.3 or not lengths:
            idle = [r for r in range(max_rows) if r not in lengths]
            rows = rng.sample(idle, min(len(idle), rng.randint(1, max(1, max_rows // 3))))
            if not rows:
                continue
            counts = [rng.randint(1, max_blocks * bs + (bs if rng.random() < 0.05 else 0)) for _ in rows]
            dev.reserve(rows, counts)
            ref.reserve(rows, counts)
            for r, c in zip(rows, counts):
                if ref.row_pages(r):
                    lengths[r] = min(c, len(ref.row_pages(r)) * bs)
        elif op < 0.8:
            rows = list(lengths)
            rng.shuffle(rows)
            pos = [lengths[r] for r in rows]
            rows_t, pos_t = torch.tensor(rows, device=DEV), torch.tensor(pos, dtype=torch.int32, device=DEV)
            if step % 2:
                dev.ensure_decode(rows_t, pos_t)
                ref.ensure_decode(rows, pos)
            else:  # the combined call: pages, then the table of the same rows
                scratch = bool(step % 4)
                got = dev.decode_step(rows_t, pos_t, pad="scratch" if scratch else "last")
                ref.ensure_decode(rows, pos)
                assert got.cpu().tolist() == ref.gather(rows, scratch, pos)
            for r in rows:
                if len(ref.row_pages(r)) * bs > lengths[r]:
                    lengths[r] += 1
        else:
            rows = rng.sample(list(lengths), rng.randint(1, len(lengths)))
            if rng.random() < 0.3:
                rows = rows + rows[:1]  # a row named twice gives its pages back once
            dev.release(rows)
            ref.release(rows)
            for r in set(rows):
                del lengths[r]
        _same_state(dev, ref)
        if ref.status != OK and rng.random() < 0.5:
            dev.clear_status()
            ref.status, ref.first_fail = OK, -1
        # the rectangular views of a random subset, both paddings
        if lengths:
            rows = rng.sample(list(lengths), min(len(lengths), 17)) + [-1]
            for scratch in (False, True):
                got = dev.block_table(rows, pad="scratch" if scratch else "last").cpu().tolist()
                assert got == ref.gather(rows, scratch)
    _same_state(dev, ref)


def test_exhaustion_is_recorded_and_raised_like_the_reference():
    dev = DeviceBlockTables(5, 4, 8, 4, DEV)
    ref = RefBlockTables(5, 4, 8, 4)
    dev.reserve([0, 1, 2], [8, 16, 4])
    ref.reserve([0, 1, 2], [8, 16, 4])
    _same_state(dev, ref)
    assert dev.status() == (EXHAUSTED, 1) and dev.row_pages(1) == [2, 3, 4] and dev.row_pages(2) == []
    with pytest.raises(RuntimeError, match="paged KV cache exhausted"):
        dev.check()
    full = DeviceBlockTables(9, 1, 2, 2, DEV)
    full.reserve([0], [7])
    assert full.row_pages(0) == [0, 1] and full.status() == (ROW_FULL, 0)
    bad = DeviceBlockTables(9, 2, 4, 2, DEV)
    bad.reserve([0, 5, 0], [2, 2, 4])
    assert bad.row_pages(0) == [0] and bad.status() == (BAD_ROW, 1)


def test_a_decode_step_on_a_dry_pool_touches_no_live_page():
    """Rows whose next token opens a page while the pool is empty: the step's table parks them on the scratch page, so
    the decode op's append lands there and every page that holds live tokens keeps its bytes (the reference raises
    before it decodes, rollout_state.py:222-224; a device-side step reports through the status word instead)."""
    from areno_amd.accel import attention as ops

    bs, hkv, d, rows = 4, 2, 64, 3
    num_pages = 6
    dev = DeviceBlockTables(num_pages, rows, 8, bs, DEV)
    dev.reserve([0, 1, 2], [8, 8, 6])  # 2 + 2 + 2 pages: the pool is empty; rows 0 and 1 are at a page border
    assert dev.free_count() == 0 and dev.status() == (OK, -1)
    g = torch.Generator(device=DEV).manual_seed(3)
    k_cache = torch.randn(num_pages + 1, bs, hkv, d, device=DEV, dtype=torch.bfloat16, generator=g)  # + the scratch page
    v_cache = torch.randn_like(k_cache)
    before_k, before_v = k_cache.clone(), v_cache.clone()
    lens = torch.tensor([8, 8, 6], dtype=torch.int32, device=DEV)
    table = dev.decode_step(torch.arange(rows, device=DEV), lens)
    assert dev.status() == (EXHAUSTED, 0)
    tab = table.cpu().tolist()
    assert tab[0] == [num_pages] * 8 and tab[1] == [num_pages] * 8, "unserved rows are parked on the scratch page"
    assert tab[2][:2] == dev.row_pages(2) and dev.row_pages(0) == [0, 1]
    q = torch.randn(rows, 4, d, device=DEV, dtype=torch.bfloat16, generator=g)
    ku = torch.randn(rows, hkv, d, device=DEV, dtype=torch.bfloat16, generator=g)
    vu = torch.randn_like(ku)
    ops.areno_paged_causal_attention_decode(q, ku, vu, k_cache, v_cache, table, lens)
    torch.cuda.synchronize()
    changed = (k_cache != before_k).flatten(1).any(1) | (v_cache != before_v).flatten(1).any(1)
    pages = set(torch.nonzero(changed).flatten().tolist())
    # row 2 appends at position 6 = slot 2 of its second page; the parked rows write into the scratch page only
    assert pages == {dev.row_pages(2)[1], num_pages}
    served = dev.row_pages(2)[1]
    assert torch.equal(k_cache[served, 2], ku[2]) and torch.equal(k_cache[served, :2], before_k[served, :2])
    with pytest.raises(RuntimeError, match="paged KV cache exhausted"):
        dev.check()


def test_prefill_slots_follow_the_payload_layout():
    bs = 4
    dev = DeviceBlockTables(64, 8, 10, bs, DEV)
    ref = RefBlockTables(64, 8, 10, bs)
    rows, cursors, chunks = [3, 0, 6], [0, 5, 9], [7, 1, 11]
    need = [c + n for c, n in zip(cursors, chunks)]
    dev.reserve([5], [9])  # someone else holds the first pages
    ref.reserve([5], [9])
    dev.reserve(rows, need)
    ref.reserve(rows, need)
    cu = [0]
    for n in chunks:
        cu.append(cu[-1] + n)
    ids, offs, pos = dev.prefill_slots(rows, cursors, cu, cu[-1])
    want = ref.prefill_slots(rows, cursors, chunks)
    assert ids.dtype == offs.dtype == pos.dtype == torch.int64
    assert (ids.cpu().tolist(), offs.cpu().tolist(), pos.cpu().tolist()) == want
    _same_state(dev, ref)


def test_c_abi_entry_points_and_argument_checks():
    """The same transitions through libareno_hip.so with raw pointers, and the host-side refusals."""
    nb, rows_n, mb, bs = 32, 6, 5, 8
    opts = dict(dtype=torch.int32, device=DEV)
    table, row_blocks = torch.empty(rows_n, mb, **opts), torch.empty(rows_n, **opts)
    ring, state = torch.empty(nb, **opts), torch.empty(4, **opts)
    bt = cabi.describe_block_tables(table, row_blocks, ring, state, bs)
    ref = RefBlockTables(nb, rows_n, mb, bs)
    assert cabi.block_tables_init(bt) == cabi.OK
    rows = torch.tensor([4, 1], device=DEV)
    assert cabi.block_tables_reserve(bt, rows, torch.tensor([17, 8], **opts)) == cabi.OK
    ref.reserve([4, 1], [17, 8])
    assert cabi.block_tables_ensure_decode(bt, rows, torch.tensor([24, 8], **opts)) == cabi.OK
    ref.ensure_decode([4, 1], [24, 8])
    out = torch.empty(3, mb, **opts)
    assert cabi.block_tables_gather(bt, torch.tensor([1, -1, 4], device=DEV), cabi.PAD_LAST_BLOCK, out) == cabi.OK
    assert out.cpu().tolist() == ref.gather([1, -1, 4], False)
    ids, offs = torch.empty(5, dtype=torch.int64, device=DEV), torch.empty(5, dtype=torch.int64, device=DEV)
    assert cabi.block_tables_prefill_slots(bt, torch.tensor([4], device=DEV), torch.tensor([14], **opts),
                                           torch.tensor([0, 5], **opts), 5, ids, offs) == cabi.OK  # fmt: skip
    want = ref.prefill_slots([4], [14], [5])
    assert (ids.cpu().tolist(), offs.cpu().tolist()) == want[:2]
    step_rows = torch.tensor([1, 4, -1], device=DEV)
    assert cabi.block_tables_decode_step(bt, step_rows, torch.tensor([16, 32, 0], **opts), cabi.PAD_SCRATCH_BLOCK,
                                         out) == cabi.OK  # fmt: skip
    ref.ensure_decode([1, 4, -1], [16, 32, 0])
    assert out.cpu().tolist() == ref.gather([1, 4, -1], True)
    assert state.cpu().tolist()[2:] == [ref.status, ref.first_fail] == [0, -1]  # a padded row asks for nothing
    assert cabi.block_tables_release(bt, torch.tensor([4], device=DEV)) == cabi.OK
    ref.release([4])
    s = state.cpu().tolist()
    free = [ring.cpu().tolist()[(s[0] + i) % nb] for i in range(s[1])]
    assert free == ref.free_list() and s[2:] == [ref.status, ref.first_fail]
    # refusals
    assert cabi.block_tables_gather(bt, rows, 7, out) == cabi.ERR_INVALID_ARGUMENT
    empty = cabi.BlockTables(None, None, None, None, 1, 1, 1, 1)
    assert cabi.block_tables_init(empty) == cabi.ERR_INVALID_ARGUMENT
    assert b"NULL" in cabi.lib().areno_hip_last_error()


def test_decode_step_inside_a_captured_graph():
    """The decode step's bookkeeping recorded once and replayed: the positions advance in a static buffer, pages appear as
    rows cross page borders, and every replay leaves the state the host lists reach step by step."""
    nb, n, mb, bs = 64, 5, 6, 4
    dev = DeviceBlockTables(nb, 8, mb, bs, DEV)
    ref = RefBlockTables(nb, 8, mb, bs)
    rows = [6, 2, 3, 0, 7]
    start = [3, 8, 1, 4, 11]
    dev.reserve(rows, start)
    ref.reserve(rows, start)
    rows_t = torch.tensor(rows + [-1], device=DEV)  # one padded row, as a bucketed batch has
    pos_t = torch.tensor(start + [0], dtype=torch.int32, device=DEV)
    out = torch.empty(n + 1, mb, dtype=torch.int32, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        dev.decode_step(rows_t, pos_t, pad="scratch", out=out)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    ref.ensure_decode(rows, start)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        dev.decode_step(rows_t, pos_t, pad="scratch", out=out)
    pos = list(start)
    for _ in range(9):
        pos = [p + 1 for p in pos]
        pos_t[:n] += 1
        graph.replay()
        torch.cuda.synchronize()
        ref.ensure_decode(rows, pos)
        assert out.cpu().tolist() == ref.gather(rows + [-1], True)
        _same_state(dev, ref)
