"""Decode-only steps, and steps that bring one portion of one prompt, replayed as HIP graphs.

A decode step of a small model is some hundred short kernels; launched one by
one from Python their launch cost exceeds their run time. The reference tried
to capture its decode step per batch size (lite_llama/executor/cuda_graph.py:
9-145) but its forward never takes that path (model_executor.py:314-320). Here
a step whose entries all bring one token runs through a graph captured once per
batch-size bucket: the integer tables of the step live in one static device
buffer that is refreshed by a single copy from pinned host memory, then the
graph is replayed. Rows beyond the live sequences are padding: they have
ctx_len 0 (attention reads nothing), slot -1 (nothing is written to the cache)
and their logits are dropped.

A step with a single entry of several tokens (a prompt, or a portion of one, alone in the
step: the first thing a request sees on an idle engine) is some 150 launches that cost the
host about 2.4 ms at 16 layers, more than the GPU needs for up to a thousand tokens. Such a
step runs through a graph captured once per bucket of its token count (32, 64, ... 1024):
the tokens are padded to the bucket with rows that write nothing to the cache (slot -1) and
that no query block covers (the work lists name blocks up to the bucket's size; a block
past the real tokens is empty and its workgroup leaves at once).

Nothing in a captured step clears memory with a memset node, and the buffers a
replay reads are written by ordinary copies before it.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import numpy as np
import torch

from .batch import GroupContext, StepContext, StepEntry, take_pages


def bucket_sizes(max_num_seqs: int) -> List[int]:
    out, b = [], 1
    while b < max_num_seqs:
        out.append(b)
        b *= 2
    out.append(max_num_seqs)
    return out


class _Bucket:
    """Static buffers, context and captured graph for one padded batch size."""

    def __init__(self, size: int, manager, width: int, device):
        self.size, self.width = size, width
        B, G = size, len(manager.paged)
        names = [("token_ids", B), ("positions", B), ("ctx_len", B), ("state_slots", B),
                 ("q_start", B + 1), ("logit_rows", B), ("work_off", B)]
        for g in range(G):
            names += [(f"slots{g}", B), (f"table{g}", B * width)]
        self.spans, n = {}, 0
        for name, k in names:
            self.spans[name] = (n, k)
            n += k
        self.host = torch.zeros(n, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(n, dtype=torch.int32, device=device)
        a, k = self.spans["q_start"]
        self.np[a:a + k] = np.arange(B + 1)
        a, k = self.spans["logit_rows"]
        self.np[a:a + k] = np.arange(B)
        for g in range(G):
            a, k = self.spans[f"slots{g}"]
            self.np[a:a + k] = -1
        self.table_np = [self.view_np(f"table{g}").reshape(B, width) for g in range(G)]
        self.row_owner = [[None] * B for _ in range(G)]       # (request, pages written) per row
        empty = self.dev[:0]
        # every sequence is one 16-row block at row 0: the work list of the vector-FMA
        # attention kernel, which takes the head sizes the split-KV kernel does not
        all16 = (self.view("logit_rows"), self.view("work_off"))
        groups = [GroupContext(self.view(f"table{g}").view(B, width), self.view(f"slots{g}"))
                  for g in range(G)]
        self.ctx = StepContext(
            token_ids=self.view("token_ids"), positions=self.view("positions"),
            q_start=self.view("q_start"), ctx_len=self.view("ctx_len"),
            state_slots=self.view("state_slots"), logit_rows=self.view("logit_rows"),
            work={"all16": all16, "multi16": (empty, empty), "multi64": (empty, empty),
                  "multi128": (empty, empty)},
            groups=groups,
            num_tokens=B, num_seqs=B, num_logit_rows=B, logit_rows_are_identity=True,
            num_decode_seqs=B, q_lens=[1] * B, ctx_lens=[0] * B, max_q_len=1, max_ctx_len=0)
        self.graph = None
        self.logits = None

    def view(self, name):
        a, k = self.spans[name]
        return self.dev[a:a + k]

    def view_np(self, name):
        a, k = self.spans[name]
        return self.np[a:a + k]


def capture_forward(model, storage, ctx, device):
    """(graph, logits) of one forward pass over ``ctx``, whose tensors are static buffers."""
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        model.forward(ctx, storage)                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        logits = model.forward(ctx, storage)
    return graph, logits


class DecodeGraphs:
    def __init__(self, model, manager, storage, max_model_len: int, device):
        if manager.states:
            raise ValueError("padding rows would touch state slots: models with fixed-size "
                             "state do not run through decode graphs")
        self.model, self.manager, self.storage = model, manager, storage
        self.device = device
        self.max_model_len = int(max_model_len)
        self.width = -(-self.max_model_len // manager.page_size)
        self.sizes = bucket_sizes(manager.max_num_seqs)
        self.buckets: Dict[int, _Bucket] = {}

    def fits(self, entries: Sequence[StepEntry]) -> bool:
        if len(entries) > self.sizes[-1]:
            return False
        for e in entries:
            if len(e.tokens) != 1:
                return False
            if self.manager.num_tokens.get(e.request, 0) + 1 > self.max_model_len:
                return False
        return True

    def _bucket(self, n: int) -> _Bucket:
        size = next(s for s in self.sizes if s >= n)
        b = self.buckets.get(size)
        if b is None:
            b = self.buckets[size] = _Bucket(size, self.manager, self.width, self.device)
        return b

    def _capture(self, b: _Bucket) -> None:
        # the split of the decode attention is fixed at capture: plan it for the longest context
        b.ctx.ctx_lens = [self.max_model_len] * b.size
        b.ctx.max_ctx_len = self.max_model_len
        b.graph, b.logits = capture_forward(self.model, self.storage, b.ctx, self.device)

    def step(self, entries: Sequence[StepEntry], token_feed=None) -> torch.Tensor:
        """Logits [wanted, vocab] of a step whose entries all bring one token.
        ``token_feed``: an int32 device tensor with the entries' tokens, for a step that is
        launched before the host knows them (the entries then carry placeholders)."""
        m = self.manager
        starts = take_pages(entries, m, self.model.vocab_size)
        n = len(entries)
        b = self._bucket(n)
        np_ = b.view_np
        np_("token_ids")[:n] = [e.tokens[0] for e in entries]
        np_("positions")[:n] = starts
        ctx = np_("ctx_len")
        ctx[:n] = starts
        ctx[:n] += 1
        ctx[n:] = 0
        np_("state_slots")[:n] = [m.slot_of[e.request] for e in entries]
        P = m.page_size
        for g, group in enumerate(m.paged):
            slots = np_(f"slots{g}")
            slots[n:] = -1
            table_np, owner = b.table_np[g], b.row_owner[g]
            for i, (e, pos) in enumerate(zip(entries, starts)):
                table = group.tables[e.request]
                slots[i] = table[pos // P] * P + pos % P
                have = owner[i]
                if have is not None and have[0] == e.request and have[1] <= len(table) \
                        and group.spec.window is None:
                    if have[1] < len(table):
                        table_np[i, have[1]:len(table)] = table[have[1]:]
                else:
                    table_np[i, :len(table)] = table
                owner[i] = (e.request, len(table))
        def refresh():
            b.dev.copy_(b.host, non_blocking=True)
            if token_feed is not None:
                b.view("token_ids")[:n].copy_(token_feed[:n], non_blocking=True)
        if b.graph is None:
            refresh()
            self._capture(b)
        refresh()
        b.graph.replay()
        logits = b.logits
        rows = [i for i, e in enumerate(entries) if e.want]
        if len(rows) == n and n == b.size:
            return logits
        if len(rows) == n:
            return logits[:n]
        return logits.index_select(0, torch.tensor(rows, dtype=torch.int32, device=logits.device))


PORTION_BUCKETS = (32, 64, 128, 256, 512, 1024)


class _PortionBucket:
    """Static buffers, context and captured graph for one padded token count of a
    single-entry step."""

    def __init__(self, size: int, manager, width: int, max_model_len: int, device):
        from .batch import GENERIC_BLOCK_ROWS, MFMA_BIG_BLOCK_ROWS, MFMA_BLOCK_ROWS
        self.size = T = size
        G = len(manager.paged)
        blocks = {"16": GENERIC_BLOCK_ROWS, "64": MFMA_BLOCK_ROWS, "128": MFMA_BIG_BLOCK_ROWS}
        names = [("token_ids", T), ("positions", T), ("ctx_len", 1), ("state_slots", 1),
                 ("q_start", 2), ("logit_rows", 1)]
        for tag, rows in blocks.items():
            n = -(-T // rows)
            names += [("ws_" + tag, n), ("wo_" + tag, n)]
        for g in range(G):
            names += [(f"slots{g}", T), (f"table{g}", width)]
        self.spans, n = {}, 0
        for name, k in names:
            self.spans[name] = (n, k)
            n += k
        self.host = torch.zeros(n, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(n, dtype=torch.int32, device=device)
        for tag, rows in blocks.items():               # blocks of the one sequence, last rows first
            self.view_np("wo_" + tag)[:] = np.arange(0, T, rows)[::-1]
        work = {tag: (self.view("ws_" + tag), self.view("wo_" + tag)) for tag in blocks}
        groups = [GroupContext(self.view(f"table{g}").view(1, width), self.view(f"slots{g}"))
                  for g in range(G)]
        self.ctx = StepContext(
            token_ids=self.view("token_ids"), positions=self.view("positions"),
            q_start=self.view("q_start"), ctx_len=self.view("ctx_len"),
            state_slots=self.view("state_slots"), logit_rows=self.view("logit_rows"),
            work={"all16": work["16"], "multi16": work["16"], "multi64": work["64"],
                  "multi128": work["128"]},
            groups=groups,
            num_tokens=T, num_seqs=1, num_logit_rows=1, logit_rows_are_identity=False,
            num_decode_seqs=0, q_lens=[T], ctx_lens=[max_model_len], max_q_len=T,
            max_ctx_len=max_model_len)
        self.graph = None
        self.logits = None
        self.copied = None                 # event: the last copy of ``host`` has been made

    def view(self, name):
        a, k = self.spans[name]
        return self.dev[a:a + k]

    def view_np(self, name):
        a, k = self.spans[name]
        return self.np[a:a + k]


class PortionGraphs:
    """Steps of a single entry with 2 to 1,024 tokens (and at most one wanted place)."""

    def __init__(self, model, manager, storage, max_model_len: int, device):
        if manager.states:
            raise ValueError("padding rows would touch state slots: models with fixed-size "
                             "state do not run through graphs")
        self.model, self.manager, self.storage = model, manager, storage
        self.device = device
        self.max_model_len = int(max_model_len)
        self.width = -(-self.max_model_len // manager.page_size)
        self.sizes = [s for s in PORTION_BUCKETS]
        self.buckets: Dict[int, _PortionBucket] = {}

    def fits(self, entries: Sequence[StepEntry]) -> bool:
        if len(entries) != 1:
            return False
        e = entries[0]
        n = len(e.tokens)
        return (2 <= n <= self.sizes[-1] and len(e.want) <= 1
                and self.manager.num_tokens.get(e.request, 0) + n <= self.max_model_len)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits [wanted, vocab] (one row or none) of a step with one entry."""
        m = self.manager
        tokens_of: list = []
        start = take_pages(entries, m, self.model.vocab_size, tokens_of)[0]
        e, toks = entries[0], tokens_of[0]
        n = len(toks)
        size = next(s for s in self.sizes if s >= n)
        b = self.buckets.get(size)
        if b is None:
            b = self.buckets[size] = _PortionBucket(size, m, self.width, self.max_model_len,
                                                    self.device)
        # Portions without a wanted place are not waited for, so the host can be steps ahead of
        # the GPU: the pinned buffer is written again only when its last copy has been made.
        if b.copied is not None:
            b.copied.synchronize()
        np_ = b.view_np
        np_("token_ids")[:n] = toks
        np_("token_ids")[n:] = 0
        np_("positions")[:n] = np.arange(start, start + n)
        np_("positions")[n:] = 0
        np_("q_start")[:] = (0, n)
        np_("ctx_len")[0] = start + n
        np_("state_slots")[0] = m.slot_of[e.request]
        np_("logit_rows")[0] = e.want[0] if e.want else n - 1
        for g, group in enumerate(m.paged):
            slots = np_(f"slots{g}")
            slots[:n] = m.slot_array(e.request, g, start, n)
            slots[n:] = -1
            table = group.tables[e.request]
            row = np_(f"table{g}")
            row[:len(table)] = table
            row[len(table):] = -1
        b.dev.copy_(b.host, non_blocking=True)
        if b.graph is None:
            b.graph, b.logits = capture_forward(self.model, self.storage, b.ctx, self.device)
            b.dev.copy_(b.host, non_blocking=True)
            b.copied = torch.cuda.Event()
        b.copied.record()
        b.graph.replay()
        # (the logits are the graph's own buffer: the next replay of this bucket overwrites them)
        return b.logits.clone() if e.want else b.logits[:0]
