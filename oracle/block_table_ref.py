"""Host restatement of the reference's paged-KV page bookkeeping.  TEST INFRASTRUCTURE ONLY.

Follows the list-based state of ``InferenceBatchState`` in the reference:

* free list ``list(range(num_cache_blocks))``, pages taken with ``pop(0)`` and
  given back with ``extend(blocks)``  (``areno/engine/data/rollout_state.py:55,151,225``,
  ``areno/engine/inference.py:651-658``),
* prefill admission: a row grows to ``ceil((cursor + chunk) / block_size)`` pages
  (``rollout_state.py:128-151``),
* decode: a running row whose next position starts a page gets one
  (``rollout_state.py:212-225``),
* rectangular tables padded with the row's last page (``rollout_state.py:282-285``,
  ``inference.py:573-580``) or with the scratch page id ``num_blocks``
  (``areno/engine/runtime/decode_graph.py:95,163-174``),
* per-token page id / slot / position of a packed prefill chunk (``rollout_state.py:141-149``).

Pinned by the values the reference's own test holds for this state
(``tests/test_inference_scheduler_cpu.py:135-156`` there: one two-token prompt, page size 4, two pages ->
``{0: [0]}``, free ``[1]``, then position 4 -> ``{0: [0, 1]}``) and by conservation / FIFO-order properties
(``tests/test_block_table_oracle_cpu.py``).

Where the reference raises ("paged KV cache exhausted ..."), this restatement records the status and the index of
the request instead, after the same partial allocation the reference's loop has made by then, and serves no later
request of the call -- the state a caller that catches the exception would see.
"""

from __future__ import annotations

OK, EXHAUSTED, ROW_FULL, BAD_ROW = 0, 1, 2, 3


class RefBlockTables:
    def __init__(self, num_blocks: int, max_rows: int, max_blocks: int, block_size: int):
        self.num_blocks = num_blocks
        self.max_rows = max_rows
        self.max_blocks = max_blocks
        self.block_size = block_size
        self.free = list(range(num_blocks))
        self.rows: dict[int, list[int]] = {}
        self.status = OK
        self.first_fail = -1

    def _report(self, status: int, index: int) -> None:
        self.status = max(self.status, status)
        if self.first_fail < 0 or index < self.first_fail:
            self.first_fail = index

    def _clip(self, required: int, index: int) -> int:
        if required > self.max_blocks:
            self._report(ROW_FULL, index)
            required = self.max_blocks
        return required

    def _grow(self, row: int, required: int, index: int) -> bool:
        blocks = self.rows.setdefault(row, [])
        while len(blocks) < required:
            if not self.free:
                self._report(EXHAUSTED, index)
                if not blocks:
                    del self.rows[row]
                return False
            blocks.append(self.free.pop(0))
        if not blocks:
            del self.rows[row]
        return True

    def reserve(self, rows: list[int], token_counts: list[int]) -> None:
        seen = set()
        alive = True
        for i, (row, tokens) in enumerate(zip(rows, token_counts, strict=True)):
            if not 0 <= row < self.max_rows or row in seen:
                self._report(BAD_ROW, i)
                continue
            seen.add(row)
            required = self._clip(-(-tokens // self.block_size) if tokens > 0 else 0, i)
            if alive:
                alive = self._grow(row, required, i)
            elif required > len(self.rows.get(row, [])):
                self._report(EXHAUSTED, i)

    def ensure_decode(self, rows: list[int], next_positions: list[int]) -> None:
        seen = set()
        alive = True
        for i, (row, pos) in enumerate(zip(rows, next_positions, strict=True)):
            if row < 0:  # a padded row of a bucketed decode batch (runtime/decode_graph.py:163-174)
                continue
            if row >= self.max_rows:
                self._report(BAD_ROW, i)
                continue
            if row in seen:
                continue
            seen.add(row)
            if pos < 0 or pos % self.block_size != 0 or row not in self.rows:
                continue
            required = self._clip(pos // self.block_size + 1, i)
            if alive:
                alive = self._grow(row, required, i)
            elif required > len(self.rows[row]):
                self._report(EXHAUSTED, i)

    def release(self, rows: list[int]) -> None:
        for i, row in enumerate(rows):
            if not 0 <= row < self.max_rows:
                self._report(BAD_ROW, i)
                continue
            blocks = self.rows.pop(row, None)
            if blocks:
                self.free.extend(blocks)

    def gather(self, rows: list[int], pad_scratch: bool, next_positions: list[int] | None = None) -> list[list[int]]:
        """``next_positions`` (the table of a decode step): a row without a page for the position it writes next -- the
        reference has raised by then (rollout_state.py:222-224); a device-side step cannot -- is parked on the scratch
        page, so that its token cannot land in a page that holds live tokens."""
        out = []
        for i, row in enumerate(rows):
            blocks = self.rows.get(row) if 0 <= row < self.max_rows else None
            if row >= self.max_rows or (row >= 0 and not blocks):
                self._report(BAD_ROW, i)
            if blocks and next_positions is not None and next_positions[i] >= len(blocks) * self.block_size:
                blocks = None
            if not blocks:
                out.append([self.num_blocks] * self.max_blocks)
                continue
            pad = self.num_blocks if pad_scratch else blocks[-1]
            out.append(blocks + [pad] * (self.max_blocks - len(blocks)))
        return out

    def prefill_slots(self, rows: list[int], cursors: list[int], lengths: list[int]):
        ids, offs, positions = [], [], []
        for i, (row, cursor, n) in enumerate(zip(rows, cursors, lengths, strict=True)):
            blocks = self.rows.get(row, []) if 0 <= row < self.max_rows else []
            for pos in range(cursor, cursor + n):
                col = pos // self.block_size
                if col < len(blocks):
                    ids.append(blocks[col])
                else:
                    ids.append(self.num_blocks)
                    self._report(BAD_ROW, i)
                offs.append(pos % self.block_size)
                positions.append(pos)
        return ids, offs, positions

    # ---- views used by the checks -----------------------------------------------------------------------------------
    def free_list(self) -> list[int]:
        return list(self.free)

    def row_pages(self, row: int) -> list[int]:
        return list(self.rows.get(row, []))
