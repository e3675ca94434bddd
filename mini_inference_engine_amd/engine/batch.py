"""One step's batch as data: rows of (request, its next tokens), flattened.

The reference builds three device tensors and per-portion masks with Python
loops per token (inference_engine/engine.py:133-179).  Here a step is described
by a handful of int32 arrays that live in one arena with fixed device addresses
(so a captured decode step can be replayed on them), filled with vectorised host
code and sent with one copy.  Single-token rows come first, then longer portions
(inference_engine/engine.py:137); every row, whatever its length, reads the
cache through its block table, so no mask or gathered context exists.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch


@dataclass
class StepRow:
    """A request's share of one step."""
    cache: object                    # cache.RequestCache: block tables and state slot
    tokens: Sequence[int]            # the tokens to run now
    start: int                       # position of tokens[0] = tokens of the request already in the cache
    want: Sequence[int] = ()         # offsets into ``tokens`` whose logits are wanted
    taken_from: int = -1             # >= 0: the row's one token is that entry of the tokens the last step chose
                                     # (still on the device); ``tokens`` then holds a placeholder


@dataclass
class GroupStep:
    """Per page group: where this step's tokens go and where each row's pages are."""
    block_tables: torch.Tensor       # [rows, max_blocks] int32, 0 beyond a row's pages
    slot_mapping: torch.Tensor       # [T] int32: page * page_size + position % page_size
    max_blocks: int = 0


@dataclass
class StepContext:
    num_tokens: int
    num_rows: int
    num_decode_rows: int             # leading rows of exactly one token
    num_logits: int
    input_ids: torch.Tensor          # [T] int32
    positions: torch.Tensor          # [T] int32 absolute position of each token
    token_row: torch.Tensor          # [T] int32 row of each token
    row_start: torch.Tensor          # [rows + 1] int32 offsets of rows in the flat token dim
    row_position: torch.Tensor       # [rows] int32 position of each row's first token
    row_context: torch.Tensor        # [rows] int32 keys visible after this step = position + length
    state_slots: torch.Tensor        # [rows] int32
    logit_rows: torch.Tensor         # [num_logits] int32 flat token positions, in the caller's order
    taken_from: torch.Tensor | None = None      # [T] int32, see StepRow.taken_from; -1 where input_ids holds the token
    sample_temps: torch.Tensor | None = None    # [num_logits] float32: temperature of each wanted row (0 = greedy), if
    sample_seeds: torch.Tensor | None = None    # [num_logits] int64    the step's caller wants tokens chosen from its
    sample_counters: torch.Tensor | None = None  # [num_logits] int32   logits (seed and output index of the noise stream)
    earlier_tokens: torch.Tensor | None = None  # int32: the tokens the last step chose (set by the runner)
    groups: list = field(default_factory=list)
    page_size: int = 0
    max_row_tokens: int = 0          # longest row (host)
    max_context: int = 0             # largest row_context (host), or a static bound when captured
    host: dict = field(default_factory=dict)   # the same arrays as numpy, for parts that plan on the host


class StepArena:
    """Fixed-address int32 storage for step metadata, with a pinned host mirror."""

    def __init__(self, max_tokens: int, max_rows: int, max_blocks: int, num_groups: int, device):
        self.max_tokens, self.max_rows, self.max_blocks, self.num_groups = max_tokens, max_rows, max_blocks, num_groups
        self.device = torch.device(device)
        fields_ = [("input_ids", max_tokens), ("taken_from", max_tokens), ("positions", max_tokens), ("token_row", max_tokens),
                   ("logit_rows", max_tokens), ("row_start", max_rows + 1), ("row_position", max_rows),
                   ("row_context", max_rows), ("state_slots", max_rows),
                   # what choosing a token from a row's logits needs: they travel with the step's other arrays
                   ("sample_temps", max_rows), ("sample_counters", max_rows), ("sample_seeds", 2 * max_rows)]
        for g in range(num_groups):
            fields_.append((f"slot_mapping{g}", max_tokens))
        for g in range(num_groups):
            fields_.append((f"block_tables{g}", max_rows * max_blocks))
        self.offsets, off = {}, 0
        for name, n in fields_:
            self.offsets[name] = (off, n)
            off += (n + 3) // 4 * 4          # keep every array 16-byte aligned
        self.tables_begin = self.offsets["block_tables0"][0] if num_groups else off
        self.size = off
        pin = self.device.type == "cuda"
        self.host = torch.zeros(off, dtype=torch.int32, pin_memory=pin)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(off, dtype=torch.int32, device=self.device) if pin else self.host
        self._copied = None

    def host_view(self, name: str) -> np.ndarray:
        o, n = self.offsets[name]
        return self.host_np[o:o + n]

    def dev_view(self, name: str, n: int | None = None) -> torch.Tensor:
        o, cap = self.offsets[name]
        return self.dev[o:o + (cap if n is None else n)]

    def upload(self, table_rows: int) -> None:
        """One copy of everything before the block tables plus the used rows of the tables."""
        if self.dev is self.host:
            return
        end = self.tables_begin
        self.dev[:end].copy_(self.host[:end], non_blocking=True)
        for g in range(self.num_groups):
            o, _ = self.offsets[f"block_tables{g}"]
            n = table_rows * self.max_blocks
            self.dev[o:o + n].copy_(self.host[o:o + n], non_blocking=True)
        self._copied = torch.cuda.Event()
        self._copied.record()

    def wait_uploaded(self) -> None:
        if self._copied is not None:
            self._copied.synchronize()


def order_rows(rows: Sequence[StepRow]) -> list[int]:
    """Single-token rows first, then longer portions; stable."""
    return [i for i, r in enumerate(rows) if len(r.tokens) == 1] + \
           [i for i, r in enumerate(rows) if len(r.tokens) != 1]


def build_step(rows: Sequence[StepRow], arena: StepArena, page_size: int, *, pad_rows_to: int = 0,
               static_context: int = 0, want_all: bool = False, sampling=None, pad_portion_to: int = 0) -> StepContext:
    """Flatten ``rows`` into ``arena``.  ``pad_rows_to`` adds scratch rows (one token at
    position 0, page 0, slot 0) up to a captured batch size.  ``pad_portion_to`` (one row only) lengthens the
    row to a captured number of tokens: token 0 at the positions that follow, written to the scratch page, which
    is also what the row's block table names beyond its own pages; no token of the row itself looks at them (they
    come later), and what they compute is nobody's.  ``want_all`` asks for the logits
    of every token in flat order (what a captured step produces) instead of the rows' wants.
    ``sampling``: (temperatures, seeds, counters), one entry for each wanted row of logits in their order
    (with ``want_all``: one for each of ``rows``; scratch rows are greedy), for a step whose tokens are
    chosen on the device."""
    arena.wait_uploaded()           # the last step's copy may still be reading the host mirror
    order = order_rows(rows)
    n_rows = len(rows)
    lens = np.fromiter((len(rows[i].tokens) for i in order), dtype=np.int64, count=n_rows)
    if pad_portion_to:
        if n_rows != 1 or pad_rows_to or pad_portion_to < lens[0]:
            raise ValueError(f"padding to {pad_portion_to} tokens is for one row of at most as many, without padding rows")
        lens[0] = pad_portion_to
    total_rows = max(n_rows, pad_rows_to)
    if total_rows == 0 or (lens <= 0).any():
        raise ValueError("a step needs at least one row and every row at least one token")
    pad = total_rows - n_rows
    T = int(lens.sum()) + pad
    if T > arena.max_tokens or total_rows > arena.max_rows:
        raise ValueError(f"step of {T} tokens in {total_rows} rows exceeds the arena "
                         f"({arena.max_tokens} tokens, {arena.max_rows} rows)")
    if pad and (lens != 1).any():
        raise ValueError("only steps of single-token rows can be padded")
    starts = np.fromiter((rows[i].start for i in order), dtype=np.int64, count=n_rows)
    num_decode = int((lens == 1).sum()) + pad
    # rows: decode rows, padding rows (also single tokens), then portions
    row_len = np.concatenate([lens[:num_decode - pad], np.ones(pad, np.int64), lens[num_decode - pad:]])
    row_pos = np.concatenate([starts[:num_decode - pad], np.zeros(pad, np.int64), starts[num_decode - pad:]])
    src = list(order[:num_decode - pad]) + [None] * pad + list(order[num_decode - pad:])
    row_start = np.zeros(total_rows + 1, dtype=np.int64)
    np.cumsum(row_len, out=row_start[1:])
    token_row = np.repeat(np.arange(total_rows), row_len)
    positions = np.arange(T) - row_start[token_row] + row_pos[token_row]
    ctx = row_pos + row_len
    blocks_needed = int(-(-int(ctx.max()) // page_size))
    if blocks_needed > arena.max_blocks:
        raise ValueError(f"a row needs {blocks_needed} pages; the arena holds {arena.max_blocks} per row")

    ids = arena.host_view("input_ids")
    taken = arena.host_view("taken_from")
    taken[:T] = -1
    slots_state = arena.host_view("state_slots")
    new_row_of = {}
    for r, i in enumerate(src):
        a, b = row_start[r], row_start[r + 1]
        if i is None:
            ids[a:b] = 0
            slots_state[r] = 0
        else:
            if rows[i].taken_from >= 0:
                if b - a != 1:
                    raise ValueError("only a single-token row can take its token from the last step's choices")
                ids[a] = 0
                taken[a] = rows[i].taken_from
            else:
                real = len(rows[i].tokens)
                ids[a:a + real] = rows[i].tokens
                ids[a + real:b] = 0
            slots_state[r] = rows[i].cache.state_slot
            new_row_of[i] = r
    arena.host_view("positions")[:T] = positions
    arena.host_view("token_row")[:T] = token_row
    arena.host_view("row_start")[:total_rows + 1] = row_start
    arena.host_view("row_position")[:total_rows] = row_pos
    arena.host_view("row_context")[:total_rows] = ctx

    # wanted logits, in the caller's order of rows and of ``want``
    wanted = list(range(T)) if want_all else []
    for i, r in enumerate(rows if not want_all else ()):
        base = row_start[new_row_of[i]]
        for w in r.want:
            if not 0 <= w < len(r.tokens):
                raise ValueError(f"wanted offset {w} outside a row of {len(r.tokens)} tokens")
            wanted.append(base + w)
    R = len(wanted)
    arena.host_view("logit_rows")[:R] = wanted
    if sampling is not None:
        temps, seeds, counters = sampling
        n = len(temps)
        if not (len(seeds) == len(counters) == n) or n != (n_rows if want_all else R) or R > arena.max_rows:
            raise ValueError(f"sampling inputs for {n} rows; the step has {n_rows if want_all else R} rows of wanted "
                             f"logits (at most {arena.max_rows})")
        ht, hc, hs = arena.host_view("sample_temps"), arena.host_view("sample_counters"), arena.host_view("sample_seeds")
        ht[:R], hc[:R], hs[:2 * R] = 0, 0, 0
        ht[:n] = np.asarray(temps, dtype=np.float32).view(np.int32)
        hc[:n] = np.asarray(counters, dtype=np.int32)
        hs[:2 * n] = np.asarray([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64).view(np.int32)

    mb = arena.max_blocks
    for g in range(arena.num_groups):
        bt = arena.host_view(f"block_tables{g}")[:total_rows * mb].reshape(total_rows, mb)
        width = blocks_needed
        bt[:, :width] = 0
        for r, i in enumerate(src):
            if i is None:
                continue
            t = rows[i].cache.tables[g]
            need = -(-int(row_pos[r] + (len(rows[i].tokens) if pad_portion_to else row_len[r])) // page_size)
            if len(t) < need:
                raise ValueError(f"row {i}: {len(t)} pages reserved in group {g}, {need} needed")
            bt[r, :need] = t[:need]
        page_of = bt[token_row, positions // page_size].astype(np.int64)
        if pad_portion_to:                              # padding tokens: the scratch page, also where the row's last page has room
            page_of[len(rows[0].tokens):] = 0
        arena.host_view(f"slot_mapping{g}")[:T] = page_of * page_size + positions % page_size

    arena.upload(total_rows)
    step = StepContext(
        num_tokens=T, num_rows=total_rows, num_decode_rows=num_decode, num_logits=R,
        input_ids=arena.dev_view("input_ids", T), taken_from=arena.dev_view("taken_from", T),
        positions=arena.dev_view("positions", T),
        token_row=arena.dev_view("token_row", T), row_start=arena.dev_view("row_start", total_rows + 1),
        row_position=arena.dev_view("row_position", total_rows), row_context=arena.dev_view("row_context", total_rows),
        state_slots=arena.dev_view("state_slots", total_rows), logit_rows=arena.dev_view("logit_rows", R),
        page_size=page_size, max_row_tokens=int(row_len.max()),
        max_context=int(static_context or ctx.max()),
        host={"row_start": row_start, "row_position": row_pos, "row_context": ctx, "row_len": row_len,
              "positions": positions, "token_row": token_row, "state_slots": slots_state[:total_rows].copy()},
    )
    if sampling is not None:
        step.sample_temps = arena.dev_view("sample_temps", R).view(torch.float32)
        step.sample_counters = arena.dev_view("sample_counters", R)
        step.sample_seeds = arena.dev_view("sample_seeds", 2 * R).view(torch.int64)
    for g in range(arena.num_groups):
        step.groups.append(GroupStep(
            block_tables=arena.dev_view(f"block_tables{g}", total_rows * mb).view(total_rows, mb),
            slot_mapping=arena.dev_view(f"slot_mapping{g}", T), max_blocks=mb))
    return step
