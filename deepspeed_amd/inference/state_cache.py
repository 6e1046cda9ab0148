"""Paged per-token rows + per-slot carried state for ragged serving batches.

``PagedKVCache`` (ragged.py) stores K and V per head and hands the model
padded views. Models whose mixers cache something else — a compressed latent
row per token, the last few inputs of a short convolution — need two kinds
of storage that this manager provides side by side:

* **row pools**: for every cache *stream* (one per layer run) a tensor
  ``[num_blocks, block_size, row_dim]``. A sequence owns a growing list of
  blocks; all streams share one block table, so block ``b`` means the same
  token range in every stream.
* **slot states**: fixed-size tensors per request slot (``[num_slots, ...]``)
  for state that does not grow with the sequence. They are cleared when a
  slot is handed out again.

A step is described by a ``RaggedBatch``: the flat token list of several
sequences, each contributing ``count`` new tokens after the ``start`` tokens
it already holds. Kernels index the pools through ``tok_row`` (where a new
token's row is written) and ``block_table`` (where a sequence's history
lives); no padded copy of the history is made.
"""

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class RaggedBatch:
    """One step's flat batch. Device tensors are int32."""
    slots: List[int]
    starts: List[int]
    counts: List[int]
    n_tokens: int
    max_ctx: int
    block_size: int
    cu: torch.Tensor            # [n+1] first flat token of each sequence
    seq_slot: torch.Tensor      # [n]
    seq_start: torch.Tensor     # [n] tokens held before this step
    tok_seq: torch.Tensor       # [T] entry index of each token
    tok_pos: torch.Tensor       # [T] absolute position
    tok_row: torch.Tensor       # [T] block * block_size + offset in the pools
    block_table: torch.Tensor   # [n, max_blocks]
    extra: Dict = field(default_factory=dict)   # per-op work lists, cached

    @property
    def n_seqs(self) -> int:
        return len(self.slots)

    def last_token_rows(self) -> List[int]:
        out, at = [], 0
        for c in self.counts:
            at += c
            out.append(at - 1)
        return out


class PagedStateCache:
    def __init__(self, row_dims: Sequence[int], state_shapes: Dict[str, tuple],
                 num_slots: int, max_tokens: int, block_size: int = 64,
                 dtype=torch.float32, device="cpu"):
        """``row_dims[i]`` is the row width of stream ``i``;
        ``state_shapes[name]`` the per-slot shape of a carried state, or
        ``(shape, dtype)`` for a state kept in another number format than
        the pools (a recurrence's fp32 matrix beside 16-bit rows).
        ``max_tokens`` bounds the tokens live at once (each sequence rounded
        up to whole blocks)."""
        self.block_size = block_size
        self.num_blocks = max(1, (max_tokens + block_size - 1) // block_size)
        self.num_slots = num_slots
        self.device = torch.device(device)
        self.dtype = dtype
        self.pools = [torch.zeros(self.num_blocks, block_size, d, dtype=dtype,
                                  device=device) for d in row_dims]
        self.states = {}
        for k, s in state_shapes.items():
            sdt = dtype
            if len(s) == 2 and isinstance(s[1], torch.dtype):
                s, sdt = s
            self.states[k] = torch.zeros((num_slots,) + tuple(s), dtype=sdt,
                                         device=device)
        self.free_blocks = list(range(self.num_blocks - 1, -1, -1))
        self.block_table: Dict[int, List[int]] = {s: [] for s in
                                                  range(num_slots)}
        self.lens = torch.zeros(num_slots, dtype=torch.long)   # host side
        self.max_seq = self.num_blocks * block_size
        self.batch: Optional[RaggedBatch] = None

    # ------------------------------------------------------------ slots
    def free(self, slot: int):
        """Give a slot's blocks back. The rows keep their old contents; a new
        owner overwrites a row before any of its queries can see it."""
        self.free_blocks.extend(reversed(self.block_table[slot]))
        self.block_table[slot] = []
        self.lens[slot] = 0

    def reset_slot(self, slot: int):
        """Prepare a slot for a new sequence: no blocks, zero carried state."""
        self.free(slot)
        for st in self.states.values():
            st[slot].zero_()

    def blocks_free(self) -> int:
        return len(self.free_blocks)

    def blocks_needed(self, slot: int, count: int) -> int:
        upto = int(self.lens[slot]) + count
        need = (upto + self.block_size - 1) // self.block_size
        return max(0, need - len(self.block_table[slot]))

    # ------------------------------------------------------------- steps
    def begin_ragged(self, slots: Sequence[int],
                     counts: Sequence[int]) -> RaggedBatch:
        bs = self.block_size
        slots, counts = list(slots), list(counts)
        assert len(set(slots)) == len(slots), "a slot appears once per step"
        starts = [int(self.lens[s]) for s in slots]
        for s, st, c in zip(slots, starts, counts):
            need = (st + c + bs - 1) // bs
            tab = self.block_table[s]
            while len(tab) < need:
                if not self.free_blocks:
                    raise RuntimeError("paged state pool exhausted")
                tab.append(self.free_blocks.pop())
        n, T = len(slots), int(sum(counts))
        maxb = max(1, max(len(self.block_table[s]) for s in slots))
        cu = np.zeros(n + 1, np.int32)
        cu[1:] = np.cumsum(counts)
        table = np.zeros((n, maxb), np.int32)
        tok_seq = np.empty(T, np.int32)
        tok_pos = np.empty(T, np.int32)
        tok_row = np.empty(T, np.int32)
        for i, (s, st, c) in enumerate(zip(slots, starts, counts)):
            tab = np.asarray(self.block_table[s], np.int32)
            table[i, :len(tab)] = tab
            pos = np.arange(st, st + c, dtype=np.int32)
            tok_seq[cu[i]:cu[i + 1]] = i
            tok_pos[cu[i]:cu[i + 1]] = pos
            tok_row[cu[i]:cu[i + 1]] = tab[pos // bs] * bs + pos % bs
        parts = [cu, np.asarray(slots, np.int32), np.asarray(starts, np.int32),
                 tok_seq, tok_pos, tok_row, table.reshape(-1)]
        flat = torch.from_numpy(np.concatenate(parts)).to(self.device)
        views, at = [], 0
        for p in parts:
            views.append(flat[at:at + p.size])
            at += p.size
        self.batch = RaggedBatch(
            slots=slots, starts=starts, counts=counts, n_tokens=T,
            max_ctx=max(st + c for st, c in zip(starts, counts)),
            block_size=bs, cu=views[0], seq_slot=views[1], seq_start=views[2],
            tok_seq=views[3], tok_pos=views[4], tok_row=views[5],
            block_table=views[6].view(n, maxb))
        return self.batch

    def end_step(self):
        b = self.batch
        for s, c in zip(b.slots, b.counts):
            self.lens[s] += c
        self.batch = None
