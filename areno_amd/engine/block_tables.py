"""Device-resident page bookkeeping for the paged KV cache.

The reference keeps the free list and every running sequence's page list as Python lists in
``InferenceBatchState`` (areno/engine/data/rollout_state.py:55-56), walks them on the host each decode step
(``ensure_decode_blocks`` l.212-225 after a device-to-host copy of the positions, areno/engine/inference.py:561-571)
and uploads a freshly built rectangular table (``_block_table_for_active_rows``, inference.py:573-580).  This class
keeps the same state in device memory and makes the same transitions with small HIP kernels in the same order, so
a row gets the page ids the reference would give it, a decode step needs no host walk, no device-to-host copy and
no table upload, and the calls can sit inside a captured decode graph.

What stays on the host is what the reference's scheduler decides from lengths alone (which prompts to admit, how
long a chunk is): those need page *counts*, which follow from lengths the host already has, not page ids.
"""

from __future__ import annotations

import torch

from areno_amd.accel._extension import extension

STATUS_OK, STATUS_EXHAUSTED, STATUS_ROW_FULL, STATUS_BAD_ROW = 0, 1, 2, 3

_MESSAGES = {
    STATUS_EXHAUSTED: "paged KV cache exhausted",  # the reference's RuntimeError text (rollout_state.py:136,224)
    STATUS_ROW_FULL: "a sequence needs more pages than max_blocks_per_seq",
    STATUS_BAD_ROW: "block-table request names a row that is out of range, repeated or not running",
}


class DeviceBlockTables:
    """Free list, per-row page lists and their rectangular views, all on ``device``.

    ``num_cache_blocks`` pages with ids ``0 .. num_cache_blocks - 1``; the id ``num_cache_blocks`` is the scratch
    page that pads captured-graph tables (areno/engine/runtime/decode_graph.py:95), so cache pools used with
    ``pad="scratch"`` tables need ``num_cache_blocks + 1`` pages.
    """

    def __init__(self, num_cache_blocks: int, max_rows: int, max_blocks_per_seq: int, block_size: int,
                 device: torch.device | str):  # fmt: skip
        if min(num_cache_blocks, max_rows, max_blocks_per_seq, block_size) <= 0:
            raise ValueError("block-table geometry must be positive")
        self.num_cache_blocks = num_cache_blocks
        self.max_rows = max_rows
        self.max_blocks_per_seq = max_blocks_per_seq
        self.block_size = block_size
        self.device = torch.device(device)
        self._ext = extension()
        opts = {"device": self.device, "dtype": torch.int32}
        self.table = torch.empty(max_rows, max_blocks_per_seq, **opts)
        self.row_blocks = torch.empty(max_rows, **opts)
        self.free_ring = torch.empty(num_cache_blocks, **opts)
        self.state = torch.empty(4, **opts)
        self.reset()

    @property
    def scratch_block(self) -> int:
        return self.num_cache_blocks

    def _args(self):
        return self.table, self.row_blocks, self.free_ring, self.state, self.block_size

    def _rows(self, rows) -> torch.Tensor:
        if not isinstance(rows, torch.Tensor):
            rows = torch.tensor(list(rows), dtype=torch.long)
        return rows.to(device=self.device, dtype=torch.long).contiguous()

    def _counts(self, values) -> torch.Tensor:
        if not isinstance(values, torch.Tensor):
            values = torch.tensor(list(values), dtype=torch.int32)
        return values.to(device=self.device, dtype=torch.int32).contiguous()

    def reset(self) -> None:
        """All pages free in id order, no row running (rollout_state.py:55-56)."""
        self._ext.areno_block_tables_init(*self._args())

    def reserve(self, rows, token_counts) -> None:
        """Prefill admission: row ``rows[i]`` must hold ``token_counts[i]`` tokens (cursor + chunk length)."""
        self._ext.areno_block_tables_reserve(*self._args(), self._rows(rows), self._counts(token_counts), False)

    def ensure_decode(self, rows, next_positions) -> None:
        """A running row whose next position (the decode op's ``cache_seqlens``) starts a page gets that page."""
        self._ext.areno_block_tables_reserve(*self._args(), self._rows(rows), self._counts(next_positions), True)

    def release(self, rows) -> None:
        """Pages of the rows go back to the tail of the free list, in row order (inference.py:651-658)."""
        self._ext.areno_block_tables_release(*self._args(), self._rows(rows))

    def block_table(self, rows, pad: str = "last", out: torch.Tensor | None = None) -> torch.Tensor:
        """``[len(rows), max_blocks_per_seq]`` int32 table for the attention ops.  ``pad="last"`` repeats a row's
        last page (eager tables), ``pad="scratch"`` writes the scratch id (graph tables); a negative row index gives
        a row of scratch ids (the padded rows of a captured batch).  ``out`` reuses a static buffer."""
        if pad not in ("last", "scratch"):
            raise ValueError("pad must be 'last' or 'scratch'")
        return self._ext.areno_block_tables_gather(*self._args(), self._rows(rows), pad == "scratch", out)

    def decode_step(self, rows, next_positions, pad: str = "last", out: torch.Tensor | None = None) -> torch.Tensor:
        """``ensure_decode`` then ``block_table`` for the same rows in one call: the per-step pair the reference
        runs on the host (inference.py:561-580)."""
        if pad not in ("last", "scratch"):
            raise ValueError("pad must be 'last' or 'scratch'")
        return self._ext.areno_block_tables_decode_step(
            *self._args(), self._rows(rows), self._counts(next_positions), pad == "scratch", out
        )

    def prefill_slots(self, rows, cursors, cu_seqlens, total_tokens: int):
        """``(cache_block_ids, cache_block_offsets, position_ids)`` of a packed prefill chunk, int64 like the
        reference's payload (rollout_state.py:141-149, 196-203)."""
        return tuple(
            self._ext.areno_block_tables_prefill_slots(
                *self._args(), self._rows(rows), self._counts(cursors), self._counts(cu_seqlens), int(total_tokens)
            )
        )

    # ---- host-visible views (each synchronises; for admission control, tests and error reporting) -------------------
    def free_count(self) -> int:
        return int(self.state[1].item())

    def status(self) -> tuple[int, int]:
        """(worst status since the last reset / clear, index of the first refused request of the call that set it)."""
        s = self.state.cpu()
        return int(s[2]), int(s[3])

    def check(self) -> None:
        """Raise like the reference does when the pool ran dry or a request was malformed."""
        status, index = self.status()
        if status != STATUS_OK:
            raise RuntimeError(f"{_MESSAGES.get(status, 'block-table error')} (request {index})")

    def clear_status(self) -> None:
        self.state[2:4] = torch.tensor([STATUS_OK, -1], dtype=torch.int32, device=self.device)

    def free_list(self) -> list[int]:
        s = self.state.cpu().tolist()
        ring = self.free_ring.cpu().tolist()
        return [ring[(s[0] + i) % self.num_cache_blocks] for i in range(s[1])]

    def row_pages(self, row: int) -> list[int]:
        n = int(self.row_blocks[row].item())
        return self.table[row, :n].cpu().tolist()
