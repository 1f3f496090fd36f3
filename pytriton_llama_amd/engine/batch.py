"""The flat batch of one step.

The reference's forward takes a padded [B, S] token matrix that is either all
prompts of one length or all single tokens, plus a shared mutable AttentionInfo
(lite_llama/executor/model_executor.py:314-320, lite_llama/executor/
executor_struct.py:12-17). Here a step is a list of (request, its next tokens,
the places whose logits are wanted), cut anywhere, and everything a kernel
needs travels in one StepContext.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

GENERIC_BLOCK_ROWS = 16   # query rows per work item of the vector-FMA attention kernel
MFMA_BLOCK_ROWS = 64      # ... of the matrix-core prefill kernel, for short portions
MFMA_BIG_BLOCK_ROWS = 128  # ... and for long ones


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
    work: dict                     # name -> (sequence int32 [W], first query row int32 [W]):
                                   # "all16": 16-row blocks of every sequence; "multi16" /
                                   # "multi64" / "multi128": 16- / 64- / 128-row blocks of the
                                   # sequences after the leading single-token ones
    groups: List[GroupContext]
    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    logit_rows_are_identity: bool
    num_decode_seqs: int           # leading sequences that bring a single token
    q_lens: List[int] = field(default_factory=list)       # host copies
    ctx_lens: List[int] = field(default_factory=list)
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


def build_context(entries: Sequence[StepEntry], manager, device, vocab_size: Optional[int] = None):
    """Take pages for every entry (all or nothing) and lay the batch out.
    Returns (StepContext, order) where ``order`` is the permutation applied to
    the entries; logit rows are listed in the caller's order of entries."""
    tokens_of: list = []
    starts = take_pages(entries, manager, vocab_size, tokens_of)

    order = order_entries(entries)
    i32 = lambda values: np.asarray(values, dtype=np.int32)
    token_ids, positions = [], []
    q_start = [0]
    ctx_len: List[int] = []
    state_slots: List[int] = []
    slots: List[list] = [[] for _ in manager.paged]
    row_of_entry = {}
    for i in order:
        e = entries[i]
        n = len(e.tokens)
        start = starts[i]
        row_of_entry[i] = q_start[-1]
        token_ids.append(tokens_of[i])
        positions.append(np.arange(start, start + n, dtype=np.int32))
        q_start.append(q_start[-1] + n)
        ctx_len.append(start + n)
        state_slots.append(manager.slot_of[e.request])
        for g in range(len(manager.paged)):
            slots[g].append(manager.slot_array(e.request, g, start, n))
    logit_rows = [row_of_entry[i] + w for i, e in enumerate(entries) for w in e.want]
    T = q_start[-1]
    nseq = len(order)
    q_lens = [q_start[i + 1] - q_start[i] for i in range(nseq)]
    num_decode = 0
    while num_decode < nseq and q_lens[num_decode] == 1:
        num_decode += 1
    work = {"all16": work_items(q_lens, ctx_len, 0, GENERIC_BLOCK_ROWS),
            "multi16": work_items(q_lens, ctx_len, num_decode, GENERIC_BLOCK_ROWS),
            "multi64": work_items(q_lens, ctx_len, num_decode, MFMA_BLOCK_ROWS),
            "multi128": work_items(q_lens, ctx_len, num_decode, MFMA_BIG_BLOCK_ROWS)}
    tables = []
    for g, group in enumerate(manager.paged):
        rows = [group.tables[entries[i].request] for i in order]
        width = max(1, max(len(r) for r in rows))
        table = np.full((nseq, width), -1, dtype=np.int32)
        for r, row in enumerate(rows):
            table[r, :len(row)] = row
        tables.append(table)

    # one host->device copy for all integer arrays
    parts: List[np.ndarray] = []
    spans = {}
    filled = 0

    def put(name, values):
        nonlocal filled
        values = i32(values).reshape(-1)
        spans[name] = (filled, values.size)
        parts.append(values)
        filled += values.size

    put("token_ids", np.concatenate(token_ids))
    put("positions", np.concatenate(positions))
    put("q_start", q_start)
    put("ctx_len", ctx_len)
    put("state_slots", state_slots)
    put("logit_rows", logit_rows)
    for name, (ws, wo) in work.items():
        put("ws_" + name, ws)
        put("wo_" + name, wo)
    for g in range(len(manager.paged)):
        put(f"slots{g}", np.concatenate(slots[g]))
        put(f"table{g}", tables[g])
    if torch.device(device).type != "cpu":
        staged = torch.empty(filled, dtype=torch.int32, pin_memory=True)
        np.concatenate(parts, out=staged.numpy())
        buf = staged.to(device, non_blocking=True)
    else:
        buf = torch.from_numpy(np.concatenate(parts))

    def get(name):
        a, n = spans[name]
        return buf[a:a + n]

    groups = [GroupContext(get(f"table{g}").view(nseq, -1), get(f"slots{g}"))
              for g in range(len(manager.paged))]
    ctx = StepContext(
        token_ids=get("token_ids"), positions=get("positions"), q_start=get("q_start"),
        ctx_len=get("ctx_len"), state_slots=get("state_slots"), logit_rows=get("logit_rows"),
        work={name: (get("ws_" + name), get("wo_" + name)) for name in work}, groups=groups,
        num_tokens=T, num_seqs=nseq, num_logit_rows=len(logit_rows),
        logit_rows_are_identity=len(logit_rows) == T and logit_rows == list(range(T)),
        num_decode_seqs=num_decode,
        q_lens=q_lens, ctx_lens=ctx_len, max_q_len=max(q_lens), max_ctx_len=max(ctx_len))
    return ctx, order
