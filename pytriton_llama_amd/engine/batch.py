"""The flat batch of one step.

The reference's forward takes a padded [B, S] token matrix that is either all
prompts of one length or all single tokens, plus a shared mutable AttentionInfo
(lite_llama/executor/model_executor.py:314-320, lite_llama/executor/
executor_struct.py:12-17). Here a step is a list of (request, its next tokens,
the places whose logits are wanted), cut anywhere, and everything a kernel
needs travels in one StepContext.

All integer arrays of a step lie in one buffer, written by one class
(StepLayout) for every way a step is run: launched kernel by kernel (the
buffer has exactly the step's size and goes to the device in one copy) and
replayed as a HIP graph (the buffer has the size of the step's size class,
lives as long as the graph, and what the step does not fill is padding). The
work lists that the model's parts ask for (parts.base.WorkList) are built here
too, for whatever block sizes they name.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import WorkList


def work_items(q_lens, ctx_lens, first_seq: int, block_rows: int):
    """(sequence, first row) of every block of ``block_rows`` query rows of the
    sequences from ``first_seq`` on, the blocks with the most keys first so
    that the long ones do not end the launch alone. Two int32 arrays."""
    seqs, offs, keys = [], [], []
    for s in range(first_seq, len(q_lens)):
        off = np.arange(0, q_lens[s], block_rows, dtype=np.int32)
        seqs.append(np.full(off.size, s, dtype=np.int32))
        offs.append(off)
        keys.append(ctx_lens[s] - q_lens[s] + np.minimum(off + block_rows, q_lens[s]))
    if not seqs:
        return np.zeros(0, dtype=np.int32), np.zeros(0, dtype=np.int32)
    seqs, offs, keys = np.concatenate(seqs), np.concatenate(offs), np.concatenate(keys)
    by_keys = np.argsort(-keys, kind="stable")
    return seqs[by_keys], offs[by_keys]


@dataclass
class StepEntry:
    """The next tokens of one request and the indices among them whose logits
    are wanted (``want`` may be empty)."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class GroupContext:
    block_table: torch.Tensor      # int32 [n, max_pages]; row i = sequence i of the batch
    slots: torch.Tensor            # int32 [T]: cache slot of every token of the batch


@dataclass
class StepContext:
    token_ids: torch.Tensor        # int32 [T]
    positions: torch.Tensor        # int32 [T]
    q_start: torch.Tensor          # int32 [n+1]: first row of every sequence
    ctx_len: torch.Tensor          # int32 [n]: tokens of the sequence in the cache after this step
    state_slots: torch.Tensor      # int32 [n]: state slot of every sequence
    logit_rows: torch.Tensor       # int32 [R]: rows whose logits are wanted
    work: Dict[WorkList, Tuple[torch.Tensor, torch.Tensor]]
                                   # the lists the model's parts asked for: WorkList ->
                                   # (sequence int32 [W], first query row int32 [W])
    groups: List[GroupContext]
    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    logit_rows_are_identity: bool
    num_decode_seqs: int           # leading sequences that bring a single token
    q_lens: List[int] = field(default_factory=list)       # host copies (in a recorded step: the
    ctx_lens: List[int] = field(default_factory=list)     # upper bounds of its size class)
    max_q_len: int = 0
    max_ctx_len: int = 0


def order_entries(entries: Sequence[StepEntry]) -> List[int]:
    """Single-token entries first (stable), so that kernels specialised for the
    decode case see one contiguous range of sequences."""
    idx = list(range(len(entries)))
    return [i for i in idx if len(entries[i].tokens) == 1] + \
           [i for i in idx if len(entries[i].tokens) != 1]


def take_pages(entries: Sequence[StepEntry], manager, vocab_size: Optional[int] = None,
               token_arrays: Optional[list] = None) -> List[int]:
    """Check the entries and take the pages for all of them, or for none.
    Returns the position of every entry's first token. ``token_arrays``: a list
    that receives every entry's tokens as an int32 array."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    for e in entries:
        if len(e.tokens) == 0:
            raise ValueError(f"request {e.request!r} brings no tokens")
        if e.request in seen:
            raise ValueError(f"request {e.request!r} appears twice in one step")
        seen.add(e.request)
        for w in e.want:
            if not 0 <= w < len(e.tokens):
                raise ValueError(f"request {e.request!r}: wanted place {w} outside its "
                                 f"{len(e.tokens)} tokens")
        if len(e.tokens) == 1 and token_arrays is None:
            bad = [] if vocab_size is None or 0 <= e.tokens[0] < vocab_size else [e.tokens[0]]
        else:
            toks = np.asarray(e.tokens)
            bad = toks[(toks < 0) | (toks >= vocab_size)] if vocab_size is not None else []
            if token_arrays is not None:
                token_arrays.append(toks.astype(np.int32, copy=False))
        if len(bad):
            raise ValueError(f"request {e.request!r}: token id {int(bad[0])} outside the "
                             f"vocabulary of {vocab_size}")
    need = [0] * len(manager.paged)
    for e in entries:
        for g, n in enumerate(manager.pages_needed(e.request, len(e.tokens))):
            need[g] += n
    for g, n in enumerate(need):
        if n > manager.paged[g].pool.num_free:
            from ..cache.manager import OutOfPages
            raise OutOfPages(f"the step needs {n} pages of group {g}, "
                             f"{manager.paged[g].pool.num_free} are free")
    return [manager.append(e.request, len(e.tokens)) for e in entries]


@dataclass(frozen=True)
class StepSizes:
    """What a step's buffer holds at most. A step launched kernel by kernel has exactly its
    own sizes; a recorded step has those of its size class."""
    decode_rows: int       # leading sequences of one token (those beyond the real ones are padding:
                           # no context, cache slot -1, the padding state slot)
    multi_seqs: int        # sequences of several tokens behind them
    multi_tokens: int      # ... and their tokens in all
    table_width: int       # pages a row of a block table names
    logit_rows: int


@dataclass
class SeqInput:
    """One sequence of a step for StepLayout.fill: its request, its tokens (an int32 array, or
    an int for a single token) and the position of the first of them."""
    request: Hashable
    tokens: object
    start: int


class StepLayout:
    """Every integer array of a step in one int32 buffer: token ids, positions, q_start,
    ctx_len, state slots, logit rows, the work lists the parts asked for, and per cache group
    the slot of every token and the block table.

    ``sizes`` fixes what the buffer holds at most; ``fill`` writes a step into it and pads
    what the step leaves: token 0 at position 0 with cache slot -1 for rows, no context and
    the manager's padding slot for single-token sequences, no rows for multi-token ones, row
    0 for logit rows, empty items for work lists. ``context`` is the StepContext over the
    device copy. A layout that is kept (for a recorded step) writes a row of a block table
    only where it grew since the last step that had the same request in that row."""

    def __init__(self, manager, work_lists: Sequence[WorkList], device, sizes: StepSizes,
                 work_items_at_most: Optional[Dict[WorkList, int]] = None):
        self.manager, self.sizes, self.device = manager, sizes, torch.device(device)
        self.work_lists = tuple(work_lists)
        B, m, T = sizes.decode_rows, sizes.multi_seqs, sizes.multi_tokens
        rows, S = B + T, B + m
        fields = [("token_ids", rows), ("positions", rows), ("q_start", S + 1), ("ctx_len", S),
                  ("state_slots", S), ("logit_rows", sizes.logit_rows)]
        for i, wl in enumerate(self.work_lists):
            most = (work_items_at_most[wl] if work_items_at_most is not None
                    else self.most_work_items(wl, sizes))
            fields += [(f"work_seq{i}", most), (f"work_row{i}", most)]
        for g in range(len(manager.paged)):
            fields += [(f"slots{g}", rows), (f"table{g}", S * sizes.table_width)]
        self.spans, n = {}, 0
        for name, k in fields:
            self.spans[name] = (n, k)
            n += k
        on_gpu = self.device.type != "cpu"
        self.host = torch.zeros(n, dtype=torch.int32, pin_memory=on_gpu)
        self.np = self.host.numpy()
        self.dev: Optional[torch.Tensor] = None     # made by ``to_device`` or by the owner
        self.np_of = {name: self.np[a:a + k] for name, (a, k) in self.spans.items()}
        self.tables_np = [self.np_of[f"table{g}"].reshape(S, sizes.table_width)
                          for g in range(len(manager.paged))]
        for t in self.tables_np:
            t[:] = -1
        # per table row: (the block table whose pages the row holds, how many of them). The
        # table is kept by identity, not by the request's name: a request that ends and comes
        # again under the same name (after a preemption, say) has a new table with other pages.
        self.row_owner = [[None] * S for _ in manager.paged]
        self.static_work = False            # work lists written once (a layout without multi-token
                                            # sequences has the same lists in every step)

    @staticmethod
    def most_work_items(wl: WorkList, sizes: StepSizes) -> int:
        blocks = -(-sizes.multi_tokens // wl.block_rows) + sizes.multi_seqs if sizes.multi_seqs else 0
        return blocks + (0 if wl.after_decode else sizes.decode_rows)

    # ---- the device side -------------------------------------------------------
    def view(self, name: str) -> torch.Tensor:
        a, k = self.spans[name]
        return self.dev[a:a + k]

    def to_device(self) -> None:
        """One host->device copy of everything (a fresh device buffer; a kept layout is
        refreshed by its owner instead)."""
        self.dev = self.host if self.device.type == "cpu" else self.host.to(self.device, non_blocking=True)

    def context(self, q_lens: List[int], ctx_lens: List[int], logit_rows_are_identity: bool) -> StepContext:
        """The StepContext over ``self.dev``. ``q_lens`` / ``ctx_lens``: the host's copies (for
        a recorded step the most its size class can bring)."""
        sz = self.sizes
        S = sz.decode_rows + sz.multi_seqs
        groups = [GroupContext(self.view(f"table{g}").view(S, sz.table_width), self.view(f"slots{g}"))
                  for g in range(len(self.manager.paged))]
        work = {wl: (self.view(f"work_seq{i}"), self.view(f"work_row{i}"))
                for i, wl in enumerate(self.work_lists)}
        return StepContext(
            token_ids=self.view("token_ids"), positions=self.view("positions"),
            q_start=self.view("q_start"), ctx_len=self.view("ctx_len"),
            state_slots=self.view("state_slots"), logit_rows=self.view("logit_rows"),
            work=work, groups=groups, num_tokens=sz.decode_rows + sz.multi_tokens, num_seqs=S,
            num_logit_rows=sz.logit_rows, logit_rows_are_identity=logit_rows_are_identity,
            num_decode_seqs=sz.decode_rows, q_lens=list(q_lens), ctx_lens=list(ctx_lens),
            max_q_len=max(q_lens, default=0), max_ctx_len=max(ctx_lens, default=0))

    # ---- writing a step ----------------------------------------------------------
    def fill(self, decode: Sequence[SeqInput], multi: Sequence[SeqInput],
             logit_rows: Sequence[int]) -> Tuple[List[int], List[int]]:
        """Write a step: ``decode`` (one token each; at most sizes.decode_rows) in rows 0..,
        ``multi`` behind row sizes.decode_rows, ``logit_rows`` (rows of the flat batch, at most
        sizes.logit_rows). The pages of all tokens have been taken. Returns the real
        (q_lens, ctx_lens) of all sequence places (padding places: 1 and 0, or 0 and 0)."""
        m, sz, A = self.manager, self.sizes, self.np_of
        B, P = sz.decode_rows, m.page_size
        k, n_multi = len(decode), len(multi)
        if k > B or n_multi > sz.multi_seqs or len(logit_rows) > sz.logit_rows:
            raise ValueError("the step is larger than its layout")
        tok, pos, ctx, slot_of, q_start = (A["token_ids"], A["positions"], A["ctx_len"],
                                           A["state_slots"], A["q_start"])
        # single-token sequences, then the padding rows up to B
        tok[:k] = [d.tokens for d in decode]
        pos[:k] = [d.start for d in decode]
        ctx[:k] = pos[:k]
        ctx[:k] += 1
        slot_of[:k] = [m.slot_of[d.request] for d in decode]
        tok[k:B] = 0
        pos[k:B] = 0
        ctx[k:B] = 0
        slot_of[k:B] = m.padding_slot
        q_start[:B + 1] = np.arange(B + 1)
        # sequences of several tokens, then places without rows, then rows that belong to nobody
        row = B
        for j, s in enumerate(multi):
            n = len(s.tokens)
            if row + n > B + sz.multi_tokens:
                raise ValueError("the step brings more tokens than its layout holds")
            tok[row:row + n] = s.tokens
            pos[row:row + n] = np.arange(s.start, s.start + n)
            row += n
            q_start[B + j + 1] = row
            ctx[B + j] = s.start + n
            slot_of[B + j] = m.slot_of[s.request]
        q_start[B + n_multi + 1:] = row
        ctx[B + n_multi:] = 0
        slot_of[B + n_multi:] = m.padding_slot
        tok[row:] = 0
        pos[row:] = 0
        lr = A["logit_rows"]
        lr[:len(logit_rows)] = logit_rows
        lr[len(logit_rows):] = 0
        for g, group in enumerate(m.paged):
            slots, table_np, owner = A[f"slots{g}"], self.tables_np[g], self.row_owner[g]
            for i, d in enumerate(decode):
                table = group.tables[d.request]
                slots[i] = table[d.start // P] * P + d.start % P
                self._table_row(table_np, owner, i, table, group.spec.window is None)
            slots[k:B] = -1
            row = B
            for j, s in enumerate(multi):
                n = len(s.tokens)
                slots[row:row + n] = m.slot_array(s.request, g, s.start, n)
                row += n
                self._table_row(table_np, owner, B + j, group.tables[s.request], False)
            slots[row:] = -1
        q_lens = [1] * B + [len(s.tokens) for s in multi] + [0] * (sz.multi_seqs - n_multi)
        ctx_lens = ctx.tolist()
        if not self.static_work:
            self._fill_work(q_lens, ctx_lens)
            self.static_work = sz.multi_seqs == 0
        return q_lens, ctx_lens

    @staticmethod
    def _table_row(table_np, owner, i: int, table: List[int], grows_only: bool) -> None:
        have = owner[i]
        if (grows_only and have is not None and have[0] is table and have[1] <= len(table)):
            if have[1] < len(table):
                table_np[i, have[1]:len(table)] = table[have[1]:]
        else:
            if len(table) > table_np.shape[1]:
                raise ValueError("a request holds more pages than a row of the layout's block table")
            table_np[i, :len(table)] = table
            table_np[i, len(table):] = -1
        owner[i] = (table, len(table))

    def _fill_work(self, q_lens: List[int], ctx_lens: List[int]) -> None:
        B = self.sizes.decode_rows
        last = len(q_lens) - 1
        for i, wl in enumerate(self.work_lists):
            ws, wo = work_items(q_lens, ctx_lens, B if wl.after_decode else 0, wl.block_rows)
            seq_np, row_np = self.np_of[f"work_seq{i}"], self.np_of[f"work_row{i}"]
            if ws.size > seq_np.size:
                raise ValueError(f"the step has {ws.size} blocks of {wl.block_rows} rows, its layout "
                                 f"holds {seq_np.size}")
            seq_np[:ws.size] = ws
            row_np[:ws.size] = wo
            if ws.size < seq_np.size:
                # empty items: the first block boundary that is not below the rows of the last
                # sequence place
                seq_np[ws.size:] = max(last, 0)
                row_np[ws.size:] = -(-max(q_lens[last] if last >= 0 else 0, 1) // wl.block_rows) * wl.block_rows


def build_context(entries: Sequence[StepEntry], manager, device, vocab_size: Optional[int] = None,
                  work_lists: Sequence[WorkList] = ()):
    """Take pages for every entry (all or nothing) and lay the batch out in a buffer of
    exactly its size. Returns (StepContext, order) where ``order`` is the permutation applied
    to the entries; logit rows are listed in the caller's order of entries."""
    tokens_of: list = []
    starts = take_pages(entries, manager, vocab_size, tokens_of)
    order = order_entries(entries)
    decode = [SeqInput(entries[i].request, int(tokens_of[i][0]), starts[i])
              for i in order if len(tokens_of[i]) == 1]
    multi = [SeqInput(entries[i].request, tokens_of[i], starts[i])
             for i in order if len(tokens_of[i]) != 1]
    row_of_entry, row = {}, 0
    for i in order:
        row_of_entry[i] = row
        row += len(tokens_of[i])
    logit_rows = [row_of_entry[i] + w for i, e in enumerate(entries) for w in e.want]
    q_lens = [1] * len(decode) + [len(s.tokens) for s in multi]
    ctx_lens = [s.start + n for s, n in zip(decode + multi, q_lens)]
    B = len(decode)
    exact = {wl: int(sum(-(-q // wl.block_rows) for q in q_lens[B if wl.after_decode else 0:]))
             for wl in work_lists}
    width = max(1, max(len(g.tables[e.request]) for g in manager.paged for e in entries)) \
        if manager.paged else 1
    sizes = StepSizes(B, len(multi), row - B, width, len(logit_rows))
    layout = StepLayout(manager, work_lists, device, sizes, exact)
    layout.fill(decode, multi, logit_rows)
    layout.to_device()
    identity = len(logit_rows) == row and logit_rows == list(range(row))
    return layout.context(q_lens, ctx_lens, identity), order
