"""Row segments of one engine step, as the sequence-mixing kernels see them.

A step's rows are [prefill chunk rows | decode rows]; every chunk and every decode row is one
SEGMENT: consecutive positions of one sequence, starting at ``start`` (the tokens the cache and
the recurrent state already hold).  The kernels need, per segment, where its rows are, which
state slot carries its sequence and which cache blocks hold its keys."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class SegBatch:
    cu: torch.Tensor          # [S + 1] int32 row offsets
    slot: torch.Tensor        # [S] int32 state slot of each segment's sequence
    start: torch.Tensor       # [S] int32 position of each segment's first row
    row_seg: torch.Tensor     # [T] int32 segment of each row
    positions: torch.Tensor   # [T] int32 position of each row in its sequence
    tables: Optional[torch.Tensor] = None   # [S, max_blocks] int32 cache blocks per segment
    cache_slots: Optional[torch.Tensor] = None  # [T] int64 cache slot of each row (-1: none)
    # prefill rows cut into tiles for the matrix-core attention kernel: [n, 2] int32 (segment,
    # first row), each tile up to TILE_ROWS rows of its segment; they cover rows [0, tile_rows)
    # (the prefill chunks; decode rows follow and take the row kernel).  None: row kernel only.
    q_tiles: Optional[torch.Tensor] = None
    tile_rows: int = 0
    tile_size: int = 64       # rows per tile of q_tiles (TILE_ROWS when they were cut)

    @property
    def S(self) -> int:
        return self.slot.shape[0]

    @property
    def T(self) -> int:
        return self.row_seg.shape[0]


import os

# rows per prefill attention tile: 128 (four waves per workgroup share a staged key tile; 167 vs
# 197 us per 4096 x 32-head x 128 call at 512-token prompts) or 64 (two)
TILE_ROWS = 64 if os.environ.get("LUMEN_ATTN_TILE_ROWS", "128") == "64" else 128


def tile_list(cu, n_segments: int, rows: int = 0):
    """[(segment, first row)] covering the first ``n_segments`` segments of row offsets ``cu``
    (host ints) in tiles of ``rows`` (default TILE_ROWS) rows."""
    rows = rows or TILE_ROWS
    return [(s, r) for s in range(n_segments) for r in range(int(cu[s]), int(cu[s + 1]), rows)]


def whole_sequences(lengths, device, slots=None, block_size: int = 16) -> SegBatch:
    """Segments for whole sequences from position 0 (one per entry of ``lengths``), with block
    tables laid out back to back: the batch a fresh forward pass runs."""
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + int(n))
    S = len(lengths)
    i32 = dict(dtype=torch.int32, device=device)
    row_seg = torch.cat([torch.full((int(n),), i, **i32) for i, n in enumerate(lengths)])
    pos = torch.cat([torch.arange(int(n), **i32) for n in lengths])
    nb = [(int(n) + block_size - 1) // block_size for n in lengths]
    tables = torch.zeros(S, max(nb), **i32)
    b0 = 0
    cache_slots = []
    for i, n in enumerate(lengths):
        tables[i, :nb[i]] = torch.arange(b0, b0 + nb[i], **i32)
        cache_slots.append(torch.arange(int(n), device=device, dtype=torch.long) + b0 * block_size)
        b0 += nb[i]
    return SegBatch(torch.tensor(cu, **i32),
                    torch.tensor(list(slots) if slots is not None else list(range(S)), **i32),
                    torch.zeros(S, **i32), row_seg, pos, tables, torch.cat(cache_slots),
                    torch.tensor(tile_list(cu, S), **i32).view(-1, 2), cu[-1], TILE_ROWS)
