"""Host-side bookkeeping of the paged sliding-window KV cache: physical block allocation,
window eviction / block recycling, slot mapping and the windowed block-table view.

In the reference this work is done by vLLM's v0 block manager and model runner (not vendored
there); the reference's own files fix the call pattern: the metadata builder takes the last
`curr_sliding_window_block` entries of each table and computes slots with
`compute_slot_mapping_start_idx` / `compute_slot_mapping`
(vllm_hymeta/attention/meta_attention.py:474-494), pads tables with 0 and slots with
PAD_SLOT_ID (:556-569), and one block table is shared by all SWA layers.

Policy of this manager (its own specification, deterministic):
  * free blocks form a LIFO stack that initially pops 0, 1, 2, ...;
  * per engine step and per sequence, in batch-row order: first evict every resident logical
    block that lies wholly before the window of the FIRST new token
    (logical block < (p0 - window_left) // block_size), lowest first, pushing each on the
    stack; then allocate, in position order, a block for every stored token whose logical
    block has none. With window_left a multiple of block_size a decoding sequence therefore
    recycles its own oldest block: a fixed ring of window_left/block_size + 1 blocks;
  * a prompt whose attention runs over the in-flight K/V stores only tokens
    i >= query_len - window_left (older ones get PAD_SLOT_ID); a prompt chunk whose attention
    reads the paged cache (chunked prefill) stores every token, because its own queries read
    them back.
Per-sequence tables are rings indexed by logical block modulo the ring size, so a step costs
O(events) Python work plus vectorised numpy, independent of the context length.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

PAD_SLOT_ID = -1


def compute_slot_mapping_start_idx(is_prompt: bool, query_len: int, context_len: int,
                                   sliding_window: Optional[int]) -> int:
    """First token index of a prompt that is cached at all (call site meta_attention.py:489-491)."""
    start_idx = 0
    if is_prompt and sliding_window is not None:
        start_idx = max(0, query_len - sliding_window)
    return start_idx


class SlotBuffer:
    """A step's slot mapping while it is being built: behaves like the reference's `slot_mapping: List[int]`
    for what the builder does with it (`extend`, `len`), but keeps what compute_slot_mapping produces as
    numpy pieces, so that a prompt step of 10^5 tokens never becomes 10^5 Python ints."""

    def __init__(self):
        self._parts: List[np.ndarray] = []
        self._n = 0

    def extend(self, values) -> None:
        a = values if isinstance(values, np.ndarray) else np.asarray(list(values), dtype=np.int64)
        if a.size:
            self._parts.append(a.astype(np.int64, copy=False))
            self._n += int(a.size)

    def __len__(self) -> int:
        return self._n

    def array(self) -> np.ndarray:
        if not self._parts:
            return np.zeros(0, dtype=np.int64)
        return self._parts[0] if len(self._parts) == 1 else np.concatenate(self._parts)

    def tolist(self) -> List[int]:
        return self.array().tolist()


def compute_slot_mapping(is_profile_run: bool, slot_mapping, seq_id, seq_len: int, context_len: int,
                         start_idx: int, block_size: int, block_tables) -> None:
    """Append one slot per new token i in [context_len, seq_len) (call site meta_attention.py:492-494):
    PAD_SLOT_ID below start_idx, else block_tables[seq_id][i // block_size] * block_size + i % block_size.
    `block_tables[seq_id]` must be indexable by ABSOLUTE logical block (a list, or the
    `LogicalTable` view of this module). `slot_mapping` is a list (as in the reference) or a SlotBuffer."""
    fast = isinstance(slot_mapping, SlotBuffer)
    if is_profile_run:
        slot_mapping.extend(np.full(seq_len, PAD_SLOT_ID, np.int64) if fast else [PAD_SLOT_ID] * seq_len)
        return
    n_pad = max(0, start_idx - context_len)
    if n_pad:
        slot_mapping.extend(np.full(n_pad, PAD_SLOT_ID, np.int64) if fast else [PAD_SLOT_ID] * n_pad)
    table = block_tables[seq_id]
    first = max(start_idx, context_len)
    if seq_len > first:
        pos = np.arange(first, seq_len, dtype=np.int64)
        jb, je = first // block_size, (seq_len - 1) // block_size
        if hasattr(table, "blocks"):
            blocks = table.blocks(jb, je)
        else:
            blocks = np.asarray([table[j] for j in range(jb, je + 1)], dtype=np.int64)
        slots = blocks[pos // block_size - jb] * block_size + pos % block_size
        slot_mapping.extend(slots if fast else slots.tolist())


class LogicalTable:
    """Read-only view of one sequence's ring as a table indexed by absolute logical block."""

    def __init__(self, mgr: "WindowBlockManager", row: int):
        self._mgr, self._row = mgr, row

    def __getitem__(self, j: int) -> int:
        m, r = self._mgr, self._row
        if j < m.lo[r] or j > m.hi[r]:
            raise IndexError(f"logical block {j} is not resident (resident {m.lo[r]}..{m.hi[r]})")
        return int(m.ring[r, j % m.ring_blocks])

    def blocks(self, jb: int, je: int) -> np.ndarray:
        """Physical blocks of logical blocks jb..je (all of them must be resident) as int64."""
        m, r = self._mgr, self._row
        if jb < m.lo[r] or je > m.hi[r]:
            raise IndexError(f"logical blocks {jb}..{je} are not all resident (resident {m.lo[r]}..{m.hi[r]})")
        return m.ring[r, np.arange(jb, je + 1) % m.ring_blocks].astype(np.int64)


class WindowBlockManager:
    """Block allocator + per-sequence window rings for up to `max_seqs` live sequences."""

    def __init__(self, num_blocks: int, block_size: int, window_left: int, max_seqs: int,
                 max_chunk_tokens: int = 0):
        if block_size % 16 != 0 or block_size < 16:
            raise ValueError(f"Invalid block size {block_size}. Must be a multiple of 16 and at least 16.")
        if window_left < 0:
            raise ValueError("window_left must be >= 0 (an unbounded window needs no eviction)")
        self.num_blocks, self.block_size, self.window_left = num_blocks, block_size, window_left
        # most blocks a sequence can hold: window + the tokens of one step, unaligned at both ends
        self.ring_blocks = (window_left + max(1, max_chunk_tokens)) // block_size + 2
        self.ring = np.zeros((max_seqs, self.ring_blocks), dtype=np.int32)
        self.n_tokens = np.zeros(max_seqs, dtype=np.int64)
        self.lo = np.zeros(max_seqs, dtype=np.int64)        # lowest resident logical block
        self.hi = np.full(max_seqs, -1, dtype=np.int64)     # highest resident logical block (-1: none)
        self._stack = np.arange(num_blocks - 1, -1, -1, dtype=np.int32)
        self._top = num_blocks                              # number of free blocks
        self._rows: Dict[object, int] = {}
        self._free_rows = list(range(max_seqs - 1, -1, -1))

    # -- sequences ------------------------------------------------------------------
    def add_seq(self, seq_id) -> int:
        if seq_id in self._rows:
            raise KeyError(f"sequence {seq_id!r} already exists")
        if not self._free_rows:
            raise RuntimeError("no free sequence row")
        r = self._free_rows.pop()
        self._rows[seq_id] = r
        self.n_tokens[r], self.lo[r], self.hi[r] = 0, 0, -1
        return r

    def free_seq(self, seq_id) -> None:
        r = self._rows.pop(seq_id)
        for j in range(int(self.lo[r]), int(self.hi[r]) + 1):
            self._push(int(self.ring[r, j % self.ring_blocks]))
        self.lo[r], self.hi[r], self.n_tokens[r] = 0, -1, 0
        self._free_rows.append(r)

    def row_of(self, seq_id) -> int:
        return self._rows[seq_id]

    @property
    def num_free_blocks(self) -> int:
        return self._top

    def free_stack(self) -> List[int]:
        """Free physical blocks, bottom of the stack first (the next allocation takes the last)."""
        return self._stack[:self._top].tolist()

    def _push(self, blk: int) -> None:
        self._stack[self._top] = blk
        self._top += 1

    def _pop(self) -> int:
        if self._top == 0:
            raise RuntimeError("out of KV cache blocks")
        self._top -= 1
        return int(self._stack[self._top])

    # -- one engine step ------------------------------------------------------------
    def _plan_row(self, r: int, count: int, is_prompt: bool, store_all: bool = False):
        """What `count` new tokens of row r evict and allocate, without touching any state (raises on a
        ring overflow): (p0, first stored position, n_evict, lo, hi after eviction, j0, n_new, new lo, new hi)."""
        bs, wl, R = self.block_size, self.window_left, self.ring_blocks
        p0 = int(self.n_tokens[r])
        lo_new = max(0, (p0 - wl) // bs)
        lo, hi = int(self.lo[r]), int(self.hi[r])
        ev_lo = lo
        n_evict = max(0, min(lo_new, hi + 1) - lo)
        if hi >= lo:
            lo = max(lo, lo_new)
            if lo > hi:  # everything evicted
                lo, hi = 0, -1
        start_idx = compute_slot_mapping_start_idx(is_prompt, count, p0, None if store_all else wl)
        first = max(p0, start_idx)
        end = p0 + count
        j0 = n_new = 0
        if end > first:
            jb, je = first // bs, (end - 1) // bs
            if hi < lo:
                lo, hi = jb, jb - 1
            if je - lo + 1 > R:
                raise RuntimeError(f"{je - lo + 1} resident blocks exceed the ring of {R}; raise max_chunk_tokens")
            j0 = max(jb, hi + 1)
            n_new = max(0, je + 1 - j0)
            hi = max(hi, je)
        return p0, first, ev_lo, n_evict, j0, n_new, lo, hi, end

    def _apply_plan(self, r: int, plan) -> Tuple[int, int]:
        """Carries a plan of `_plan_row` out; the caller has checked that the free stack covers it."""
        R = self.ring_blocks
        p0, first, ev_lo, n_evict, j0, n_new, lo, hi, end = plan
        if n_evict > 0:  # pushed in order of logical block, as one slice
            self._stack[self._top:self._top + n_evict] = self.ring[r, np.arange(ev_lo, ev_lo + n_evict) % R]
            self._top += n_evict
        if n_new > 0:  # popped one after the other from the top of the stack, as one reversed slice
            self.ring[r, np.arange(j0, j0 + n_new) % R] = self._stack[self._top - n_new:self._top][::-1]
            self._top -= n_new
        self.lo[r], self.hi[r] = lo, hi
        self.n_tokens[r] = end
        return p0, first

    def _advance_row(self, r: int, count: int, is_prompt: bool, store_all: bool = False) -> Tuple[int, int]:
        """Evict + allocate for `count` new tokens of row r; returns (p0, first stored position).
        All or nothing: when the blocks do not suffice (or the ring would overflow) it raises with the
        row, the ring and the free stack exactly as they were, so the caller may free sequences and retry."""
        plan = self._plan_row(r, count, is_prompt, store_all)
        if plan[5] > self._top + plan[3]:
            raise RuntimeError("out of KV cache blocks")
        return self._apply_plan(r, plan)

    def append_tokens(self, seq_id, count: int, is_prompt: bool, store_all: bool = False,
                      want_slots: bool = True) -> List[int]:
        """Slots of `count` new tokens of one sequence (one prompt chunk or one decode token).
        store_all=True keeps every prompt token (chunked prefill through the paged cache).
        want_slots=False only advances the sequence (the caller works the slots out from the tables)."""
        r = self._rows[seq_id]
        p0, first = self._advance_row(r, count, is_prompt, store_all)
        slots: List[int] = []
        if not want_slots:
            return slots
        compute_slot_mapping(False, slots, r, p0 + count, p0, first, self.block_size, {r: LogicalTable(self, r)})
        return slots

    def decode_step(self, seq_ids: Sequence) -> np.ndarray:
        """One new token for every sequence of `seq_ids` (batch-row order); returns slot_mapping
        int64 [len(seq_ids)]. Only rows that cross a block boundary do Python work."""
        bs, wl, R = self.block_size, self.window_left, self.ring_blocks
        rows = np.fromiter((self._rows[s] for s in seq_ids), dtype=np.int64, count=len(seq_ids))
        p = self.n_tokens[rows]
        need_evict = (np.maximum(0, (p - wl) // bs) > self.lo[rows]) & (self.hi[rows] >= self.lo[rows])
        need_alloc = (p // bs) > self.hi[rows]
        # all or nothing over the batch: plan every row that evicts or allocates, replay the free count in
        # batch-row order, and only then touch anything
        busy = [int(rows[i]) for i in np.nonzero(need_evict | need_alloc)[0]]
        plans = [self._plan_row(r, 1, False) for r in busy]
        top = self._top
        for plan in plans:
            top += plan[3]
            if plan[5] > top:
                raise RuntimeError("out of KV cache blocks")
            top -= plan[5]
        for r, plan in zip(busy, plans):
            self._apply_plan(r, plan)
        quiet = ~(need_evict | need_alloc)
        self.n_tokens[rows[quiet]] += 1
        return self.ring[rows, (p // bs) % R].astype(np.int64) * bs + p % bs

    # -- kernel view ----------------------------------------------------------------
    def kernel_view(self, seq_ids: Sequence, pad_blocks: Optional[int] = None) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
        """(block_tables int32 [B, max_blocks] padded with 0, cache_seqlens int32 [B], first resident
        position int64 [B]). Key index k of row b is absolute position first[b] + k; the newest
        token sits at index cache_seqlens[b] - 1."""
        R, bs = self.ring_blocks, self.block_size
        rows = np.fromiter((self._rows[s] for s in seq_ids), dtype=np.int64, count=len(seq_ids))
        lo, hi = self.lo[rows], self.hi[rows]
        nblk = np.maximum(hi - lo + 1, 0)
        width = int(nblk.max()) if len(rows) else 0
        if pad_blocks is not None:
            if pad_blocks < width:
                raise ValueError(f"pad_blocks {pad_blocks} < widest table {width}")
            width = pad_blocks
        j = lo[:, None] + np.arange(width, dtype=np.int64)[None, :]
        tables = np.where(j <= hi[:, None], self.ring[rows[:, None], j % R], 0).astype(np.int32)
        seqlens = np.where(nblk > 0, self.n_tokens[rows] - lo * bs, 0).astype(np.int32)
        return tables, seqlens, lo * bs


class DeviceWindowState:
    """The manager's state for a fixed decoding batch, resident on the GPU, advanced there one token
    per sequence per call (`ops.window_advance`): the device-side counterpart of
    `WindowBlockManager.decode_step` + `kernel_view`, with the same policy and therefore the same
    slots, tables and free-stack order, bit for bit. The role ops.advance_step_flashattn plays for the
    reference's multi-step decode (vllm_hymeta/attention/meta_attention.py:338-409), extended by the
    window bookkeeping, so that a run of decode steps (or a captured graph of them) does no host work.

    Built from a host manager (`upload`); `download` writes the advanced state back into it, e.g.
    before sequences join or leave the batch (membership changes stay host-side)."""

    def __init__(self, manager: WindowBlockManager, seq_ids: Sequence, device, table_width: Optional[int] = None):
        import torch

        from . import ops
        self._torch, self._ops = torch, ops
        self.manager, self.seq_ids = manager, list(seq_ids)
        self.device = torch.device(device)
        self.rows = np.fromiter((manager.row_of(s) for s in self.seq_ids), dtype=np.int64, count=len(self.seq_ids))
        B = len(self.seq_ids)
        self.table_width = manager.ring_blocks if table_width is None else int(table_width)
        if self.table_width < manager.window_left // manager.block_size + 2:
            raise ValueError("table_width cannot hold a full window")
        i32, i64 = torch.int32, torch.int64
        self.n_tokens = torch.empty(B, dtype=i64, device=self.device)
        self.lo = torch.empty(B, dtype=i32, device=self.device)
        self.hi = torch.empty(B, dtype=i32, device=self.device)
        self.ring = torch.empty(B, manager.ring_blocks, dtype=i32, device=self.device)
        self.free_stack = torch.empty(manager.num_blocks, dtype=i32, device=self.device)
        self.free_top = torch.empty(1, dtype=i32, device=self.device)
        self.slot_mapping = torch.full((B,), PAD_SLOT_ID, dtype=i64, device=self.device)
        self.seq_lens = torch.zeros(B, dtype=i32, device=self.device)
        self.block_tables = torch.zeros(B, self.table_width, dtype=i32, device=self.device)
        self.status = torch.zeros(1, dtype=i32, device=self.device)
        self.upload()

    def upload(self) -> None:
        """Host manager -> device (synchronous copies)."""
        t, m, r = self._torch, self.manager, self.rows
        self.n_tokens.copy_(t.from_numpy(m.n_tokens[r].astype(np.int64)))
        self.lo.copy_(t.from_numpy(m.lo[r].astype(np.int32)))
        self.hi.copy_(t.from_numpy(m.hi[r].astype(np.int32)))
        self.ring.copy_(t.from_numpy(np.ascontiguousarray(m.ring[r])))
        self.free_stack.copy_(t.from_numpy(m._stack))
        self.free_top.fill_(int(m._top))

    def advance(self) -> None:
        """Enqueue one decode step for every sequence on the current stream (no synchronisation)."""
        m = self.manager
        self._ops.window_advance(self.n_tokens, self.lo, self.hi, self.ring, self.free_stack, self.free_top,
                                 self.slot_mapping, self.seq_lens, self.block_tables, self.status,
                                 block_size=m.block_size, window_left=m.window_left)

    def check(self) -> None:
        """Synchronise and raise if any advance since the last check ran out of blocks or ring."""
        s = int(self.status.item())
        if s & 1:
            raise RuntimeError("out of KV cache blocks")
        if s & 2:
            raise RuntimeError("a sequence outgrew its block ring")

    def download(self) -> None:
        """Device -> host manager (synchronises)."""
        self.check()
        m, r = self.manager, self.rows
        m.n_tokens[r] = self.n_tokens.cpu().numpy()
        m.lo[r] = self.lo.cpu().numpy()
        m.hi[r] = self.hi.cpu().numpy()
        m.ring[r] = self.ring.cpu().numpy()
        m._stack[:] = self.free_stack.cpu().numpy()
        m._top = int(self.free_top.item())
