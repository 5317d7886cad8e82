"""The host restatement of the reference's page bookkeeping (oracle/block_table_ref.py), pinned by the values the
reference's own scheduler test holds and by properties its list code fixes: every page is either free or owned by
exactly one row, pages leave the free list first-in first-out, a released row's pages come back in order."""

import random

from oracle.block_table_ref import BAD_ROW, EXHAUSTED, OK, ROW_FULL, RefBlockTables


def test_values_of_the_reference_scheduler_test():
    # tests/test_inference_scheduler_cpu.py:135-156 in the reference: prompts [[1, 2]], kv_block_size 4,
    # num_cache_blocks 2 -> after prefill {0: [0]} and free [1]; ensure_decode_blocks([0], [4]) -> {0: [0, 1]}
    ref = RefBlockTables(num_blocks=2, max_rows=1, max_blocks=32, block_size=4)
    ref.reserve([0], [2])
    assert ref.rows == {0: [0]} and ref.free_list() == [1]
    ref.ensure_decode([0], [4])
    assert ref.rows == {0: [0, 1]} and ref.free_list() == [] and ref.status == OK


def test_chunked_prefill_grows_a_row_as_the_reference_does():
    # tests/test_inference_scheduler_cpu.py:110-133 there: one 5-token prompt, chunks of 2, page size 4, 2 pages
    ref = RefBlockTables(num_blocks=2, max_rows=1, max_blocks=2, block_size=4)
    for cursor, chunk, pages in ((0, 2, [0]), (2, 2, [0]), (4, 1, [0, 1])):
        ref.reserve([0], [cursor + chunk])
        assert ref.row_pages(0) == pages
        ids, offs, pos = ref.prefill_slots([0], [cursor], [chunk])
        assert pos == list(range(cursor, cursor + chunk))
        assert ids == [pages[p // 4] for p in pos] and offs == [p % 4 for p in pos]
    ref.ensure_decode([0], [5])  # position 5 does not start a page
    assert ref.row_pages(0) == [0, 1] and ref.status == OK


def _conserved(ref):
    owned = [p for pages in ref.rows.values() for p in pages]
    everything = sorted(owned + ref.free)
    assert everything == list(range(ref.num_blocks)), "a page is lost or owned twice"


def test_conservation_and_fifo_order_under_random_traffic():
    rng = random.Random(7)
    ref = RefBlockTables(num_blocks=40, max_rows=12, max_blocks=6, block_size=4)
    lengths = {}
    for _ in range(400):
        op = rng.random()
        if op < 0.3:
            rows = rng.sample(range(12), rng.randint(1, 4))
            rows = [r for r in rows if r not in lengths]
            counts = [rng.randint(1, 14) for _ in rows]
            head = ref.free_list()
            before = {r: ref.row_pages(r) for r in rows}
            ref.reserve(rows, counts)
            taken = [p for r in rows for p in ref.row_pages(r)[len(before[r]):]]
            assert taken == head[: len(taken)], "pages must leave the free list first-in first-out, in request order"
            for r, c in zip(rows, counts):
                if ref.row_pages(r):
                    lengths[r] = c
        elif op < 0.8 and lengths:
            rows = list(lengths)
            rng.shuffle(rows)
            ref.ensure_decode(rows, [lengths[r] for r in rows])
            for r in rows:
                if len(ref.row_pages(r)) * 4 > lengths[r]:
                    lengths[r] += 1
        elif lengths:
            rows = rng.sample(list(lengths), rng.randint(1, len(lengths)))
            tail = [p for r in rows for p in ref.row_pages(r)]
            ref.release(rows)
            assert ref.free_list()[len(ref.free_list()) - len(tail):] == tail, "released pages join the tail in order"
            for r in rows:
                del lengths[r]
        _conserved(ref)
    assert ref.status in (OK, EXHAUSTED, ROW_FULL)


def test_exhaustion_keeps_the_partial_allocation_and_stops_serving():
    ref = RefBlockTables(num_blocks=5, max_rows=4, max_blocks=8, block_size=4)
    ref.reserve([0, 1, 2], [8, 16, 4])  # needs 2 + 4 + 1 pages, 5 exist
    assert ref.row_pages(0) == [0, 1] and ref.row_pages(1) == [2, 3, 4] and ref.row_pages(2) == []
    assert (ref.status, ref.first_fail) == (EXHAUSTED, 1) and ref.free_list() == []
    _conserved(ref)


def test_padding_modes_and_bad_rows():
    ref = RefBlockTables(num_blocks=9, max_rows=3, max_blocks=4, block_size=2)
    ref.reserve([2, 0], [3, 7])
    assert ref.gather([0, 2], pad_scratch=False) == [[2, 3, 4, 5], [0, 1, 1, 1]]
    assert ref.gather([2, -1], pad_scratch=True) == [[0, 1, 9, 9], [9, 9, 9, 9]]
    assert ref.status == OK
    assert ref.gather([1], pad_scratch=False) == [[9, 9, 9, 9]] and ref.status == BAD_ROW  # row 1 is not running
    full = RefBlockTables(num_blocks=9, max_rows=1, max_blocks=2, block_size=2)
    full.reserve([0], [7])
    assert full.row_pages(0) == [0, 1] and full.status == ROW_FULL
    dup = RefBlockTables(num_blocks=9, max_rows=2, max_blocks=4, block_size=2)
    dup.reserve([0], [2])
    dup.ensure_decode([0, 0], [2, 2])  # the second request finds the page already there
    assert dup.row_pages(0) == [0, 1] and dup.status == OK
    dup.release([0, 0, 1])
    assert dup.free_list() == [2, 3, 4, 5, 6, 7, 8, 0, 1] and dup.status == OK
