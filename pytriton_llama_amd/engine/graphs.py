"""Decode-only steps, and steps that bring one portion of one prompt, replayed as HIP graphs.

A decode step of a small model is some hundred short kernels; launched one by
one from Python their launch cost exceeds their run time. The reference tried
to capture its decode step per batch size (lite_llama/executor/cuda_graph.py:
9-145) but its forward never takes that path (model_executor.py:314-320). Here
a step whose entries all bring one token runs through a graph captured once per
batch-size bucket: the integer tables of the step live in one static device
buffer that is refreshed by a single copy from pinned host memory, then the
graph is replayed. Rows beyond the live sequences are padding: they have
ctx_len 0 (attention reads nothing), cache slot -1 (nothing is written to the
cache pages), the manager's padding slot as state slot (a mixer with state of its own
reads and writes a row that belongs to no request) and their logits are dropped.

A step with one entry of several tokens (a prompt, or a portion of one: the first thing a
request sees on an engine that is idle or only decoding) is some 150 launches that cost the
host about 2.4 ms at 16 layers, more than the GPU needs for up to a thousand tokens. Such a
step runs through a graph captured once per bucket of its token count (32, 64, ... 512, then
every 128 up to 2,048) and
of the number of single-token entries beside it (0, 1, 2, 4, ...):
the tokens are padded to the bucket with rows that write nothing to the cache (slot -1) and
that no query block covers (the work lists name blocks up to the bucket's size; a block
past the real tokens is empty and its workgroup leaves at once). The device tensors of the
context (q_start above all) say where the real tokens end; the host copies in the context of
a recorded step (q_lens, ctx_lens and the maxima) are the bucket's upper bounds. A mixer with
state of its own must stop at q_start[i + 1], not at the padded length.

All graphs of a runner share one memory pool: they are replayed one at a time on one stream,
so what a step needs while it runs is the most that any of them needs, not the sum.

Nothing in a captured step clears memory with a memset node, and the buffers a
replay reads are written by ordinary copies before it.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

from .. import ops
from .batch import SeqInput, StepEntry, StepLayout, StepSizes, take_pages


def bucket_sizes(max_num_seqs: int) -> List[int]:
    """Numbers of decoding rows that steps are padded to: powers of two up to 32, then every 16
    (a tile of rows of the decode products: 33 to 48 rows cost less than 49 to 64), and the
    most the engine admits."""
    out, b = [], 1
    while b < max_num_seqs:
        out.append(b)
        b = b * 2 if b < 32 else b + 16
    out.append(max_num_seqs)
    return out


class _Recorded:
    """A size class of steps: the layout with its static buffers (pinned on the host, and the
    device copy a replay reads), the context over them with the host's numbers set to the most
    the class can bring, and the captured graph."""

    def __init__(self, manager, work_lists, device, sizes: StepSizes, max_model_len: int):
        self.sizes = sizes
        self.layout = StepLayout(manager, work_lists, device, sizes)
        self.layout.dev = torch.zeros_like(self.layout.host, device=device)
        B, m = sizes.decode_rows, sizes.multi_seqs
        # the split of the decode attention and the blocks of a portion are fixed at the
        # recording: planned for the longest context and the most rows
        self.ctx = self.layout.context([1] * B + [sizes.multi_tokens] * m, [max_model_len] * (B + m),
                                       logit_rows_are_identity=(m == 0))
        self.graph = None
        self.logits = None
        self.copied = None                 # event: the last copy of the pinned buffer has been made

    def wait_for_last_copy(self) -> None:
        """Steps are launched ahead of the GPU: the pinned buffer is written again only when
        its last copy to the device has been made."""
        if self.copied is not None:
            self.copied.synchronize()


def capture_forward(model, storage, ctx, device, pool=None, timed_products: bool = True):
    """(graph, logits) of one forward pass over ``ctx``, whose tensors are static buffers.
    ``pool``: the memory pool the graph's tensors come from (shared by graphs that never run
    at the same time). ``timed_products``: the library's matrix products of the step run the
    proposal that a timing of their shape keeps (timed in the warm-up pass, recorded with the
    choice); False: the library's first proposal, as in steps launched kernel by kernel."""
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), ops.timed_library_products(timed_products):
        model.forward(ctx, storage)                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=pool), ops.timed_library_products(timed_products):
        logits = model.forward(ctx, storage)
    return graph, logits


class _Graphs:
    """What the two kinds of recorded steps share: refreshing the device copy of a layout and
    recording a size class the first time a step falls into it."""

    def __init__(self, model, manager, storage, max_model_len: int, device, pool=None,
                 timed_products: bool = True):
        self.model, self.manager, self.storage = model, manager, storage
        self.device = device
        self.pool = pool
        self.timed_products = timed_products
        self.max_model_len = int(max_model_len)
        self.width = -(-self.max_model_len // manager.page_size)
        self.work_lists = tuple(model.work_lists())

    def _replay(self, b: _Recorded, refresh) -> None:
        """``refresh()`` brings the pinned buffer to the device; the graph is recorded first if
        this is the first step of its size class."""
        if b.graph is None:
            # Recording runs the step once for real beforehand. Keys and values written twice
            # are the same keys and values, but a mixer with state of its own would take the
            # step twice: while recording, every sequence's state is the padding slot's, which
            # starts from zero like a new request's.
            slot_of = b.layout.np_of["state_slots"]
            real = slot_of.copy()
            slot_of[:] = self.manager.padding_slot
            self.storage.clear_slot(self.manager.padding_slot)
            refresh()
            b.graph, b.logits = capture_forward(self.model, self.storage, b.ctx, self.device, self.pool,
                                                self.timed_products)     # waits for the device at its end
            slot_of[:] = real
            b.copied = torch.cuda.Event()
        refresh()
        b.copied.record()
        b.graph.replay()


class DecodeGraphs(_Graphs):
    """Steps whose entries all bring one token, one graph per batch-size bucket."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.sizes = bucket_sizes(self.manager.max_num_seqs)
        self.buckets: Dict[int, _Recorded] = {}

    def fits(self, entries: Sequence[StepEntry]) -> bool:
        if len(entries) > self.sizes[-1]:
            return False
        for e in entries:
            if len(e.tokens) != 1:
                return False
            if self.manager.num_tokens.get(e.request, 0) + 1 > self.max_model_len:
                return False
        return True

    def _bucket(self, n: int) -> _Recorded:
        size = next(s for s in self.sizes if s >= n)
        b = self.buckets.get(size)
        if b is None:
            b = self.buckets[size] = _Recorded(self.manager, self.work_lists, self.device,
                                               StepSizes(size, 0, 0, self.width, size), self.max_model_len)
        return b

    def step(self, entries: Sequence[StepEntry], token_feed=None) -> torch.Tensor:
        """Logits [wanted, vocab] of a step whose entries all bring one token.
        ``token_feed``: an int32 device tensor with the entries' tokens, for a step that is
        launched before the host knows them (the entries then carry placeholders)."""
        starts = take_pages(entries, self.manager, self.model.vocab_size)
        n = len(entries)
        b = self._bucket(n)
        b.wait_for_last_copy()
        # every row's logits are computed (the rows wanted are picked below)
        b.layout.fill([SeqInput(e.request, e.tokens[0], s) for e, s in zip(entries, starts)], (),
                      range(b.sizes.decode_rows))

        def refresh():
            # one short kernel reads the pinned buffer and, for a step launched ahead, the
            # tokens the step before left on the device
            ops.stage_step(b.layout.dev, b.layout.host, token_feed, b.layout.spans["token_ids"][0], n)
        self._replay(b, refresh)
        logits = b.logits
        rows = [i for i, e in enumerate(entries) if e.want]
        if len(rows) == n and n == b.sizes.decode_rows:
            return logits
        if len(rows) == n:
            return logits[:n]
        return logits.index_select(0, ops.to_device(rows, torch.int32, logits.device))


# Token counts a portion is padded to. Up to 512 tokens a step launched kernel by kernel takes
# the same time whatever its size (the host's), so coarse buckets lose nothing; beyond, the GPU
# is the bound and padding costs what it adds, so the buckets are 128 apart.
PORTION_BUCKETS = (32, 64, 128, 256, 512) + tuple(range(640, 2049, 128))
MAX_PORTION_GRAPHS = 48          # pairs of (decoding rows, portion size) kept; others run eagerly


class PortionGraphs(_Graphs):
    """Steps of single-token entries (any number up to the largest decode bucket, also none)
    and exactly one entry of 2 to 2,048 tokens with at most one wanted place."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.sizes = list(PORTION_BUCKETS)
        self.row_sizes = [0] + bucket_sizes(self.manager.max_num_seqs)
        self.buckets: Dict[tuple, _Recorded] = {}

    def _split(self, entries):
        """(indices of the single-token entries, index of the portion) or None."""
        ones, portion = [], None
        for i, e in enumerate(entries):
            if len(e.tokens) == 1:
                ones.append(i)
            elif portion is None:
                portion = i
            else:
                return None
        return None if portion is None else (ones, portion)

    def fits(self, entries: Sequence[StepEntry]) -> bool:
        split = self._split(entries)
        if split is None:
            return False
        ones, portion = split
        if len(ones) > self.row_sizes[-1]:
            return False
        e = entries[portion]
        if not (2 <= len(e.tokens) <= self.sizes[-1] and len(e.want) <= 1):
            return False
        for i in ones:
            if list(entries[i].want) not in ([], [0]):
                return False
        key = (next(r for r in self.row_sizes if r >= len(ones)),
               next(t for t in self.sizes if t >= len(e.tokens)))
        if key not in self.buckets and len(self.buckets) >= MAX_PORTION_GRAPHS:
            return False
        return all(self.manager.num_tokens.get(x.request, 0) + len(x.tokens) <= self.max_model_len
                   for x in entries)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits [wanted, vocab] in the order of the entries."""
        ones, portion = self._split(entries)
        tokens_of: list = []
        starts = take_pages(entries, self.manager, self.model.vocab_size, tokens_of)
        e, toks = entries[portion], tokens_of[portion]
        key = (next(r for r in self.row_sizes if r >= len(ones)),
               next(t for t in self.sizes if t >= len(toks)))
        b = self.buckets.get(key)
        if b is None:
            B, T = key
            b = self.buckets[key] = _Recorded(self.manager, self.work_lists, self.device,
                                              StepSizes(B, 1, T, self.width, B + 1), self.max_model_len)
        B = b.sizes.decode_rows
        b.wait_for_last_copy()
        # the logits of every single-token row and of one row of the portion are computed
        wanted_row = B + (e.want[0] if e.want else len(toks) - 1)
        b.layout.fill([SeqInput(entries[i].request, int(tokens_of[i][0]), starts[i]) for i in ones],
                      [SeqInput(e.request, toks, starts[portion])], list(range(B)) + [wanted_row])
        self._replay(b, lambda: b.layout.dev.copy_(b.layout.host, non_blocking=True))
        # rows of the graph's logits in the caller's order of entries (a copy: the next replay
        # of this bucket overwrites the graph's own buffer)
        row_of = {i: j for j, i in enumerate(ones)}
        row_of[portion] = B
        rows = [row_of[i] for i, x in enumerate(entries) if len(x.want)]
        if not rows:
            return b.logits[:0]
        return b.logits.index_select(0, ops.to_device(rows, torch.int32, b.logits.device))
