"""The container every architecture builds: embedding, blocks, final norm, head,
the cache layers the blocks use and the order in which blocks run."""
from __future__ import annotations

import fnmatch
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import ParamSource, Part, as_tensor, run_norm


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: run ``block`` with cache layer
    ``cache_layer`` (None: the block keeps nothing). ``writes`` False lets a
    block read a cache layer that another call fills. A block, and a cache
    layer, may be named by several calls."""
    block: int
    cache_layer: Optional[int]
    writes: bool = True


class CausalLM:
    """A decoder-only language model as data: parts plus a run order.

    ``prefixes`` maps every part to the checkpoint prefix of its tensors:
    a list of (prefix, part). ``ignorable`` are glob patterns of checkpoint
    tensors that may be present without being used."""

    def __init__(self, config: Any, embedding: Part, blocks: Sequence[Part], final_norm: Part,
                 head: Part, cache_layers: Sequence[object], schedule: Sequence[LayerCall],
                 prefixes: Sequence[Tuple[str, Part]], ignorable: Sequence[str] = ()):
        self.config = config
        self.embedding, self.blocks = embedding, list(blocks)
        self.final_norm, self.head = final_norm, head
        self.cache_layers = list(cache_layers)
        self.schedule = list(schedule)
        self.prefixes = list(prefixes)
        self.ignorable = tuple(ignorable)
        # called by the loader with the names of the checkpoint's tensors before it asks for
        # expected_tensors(): for what config.json leaves open and the file settles
        self.before_load = None
        for call in self.schedule:
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"run order names block {call.block}, there are {len(self.blocks)}")
            if call.cache_layer is not None and not 0 <= call.cache_layer < len(self.cache_layers):
                raise ValueError(f"run order names cache layer {call.cache_layer}, "
                                 f"there are {len(self.cache_layers)}")
        self.dtype: Optional[torch.dtype] = None
        self.device = None
        self.has_decode_copies = False

    # ---- what the loader and the builder need -------------------------------
    def expected_tensors(self) -> Dict[str, Tuple[Part, ParamSource]]:
        out: Dict[str, Tuple[Part, ParamSource]] = {}
        for prefix, part in self.prefixes:
            for src in part.param_sources():
                name = prefix + src.name
                if name in out:
                    raise ValueError(f"two parts ask for checkpoint tensor {name!r}")
                out[name] = (part, src)
        return out

    def is_ignorable(self, name: str) -> bool:
        return any(fnmatch.fnmatchcase(name, pat) for pat in self.ignorable)

    def kernel_libraries(self) -> Tuple[str, ...]:
        libs: Tuple[str, ...] = ()
        for part in [self.embedding, *self.blocks, self.final_norm, self.head]:
            libs += tuple(part.kernel_libraries)
        return tuple(dict.fromkeys(libs))

    def make_decode_copies(self) -> int:
        """Let every part build what it keeps beside its weights for faster decode steps;
        returns the bytes taken. After the weights are loaded."""
        self.has_decode_copies = True
        return sum(p.make_decode_copies() for p in [self.embedding, *self.blocks, self.final_norm, self.head]
                   if hasattr(p, "make_decode_copies"))

    def work_lists(self) -> Tuple[Any, ...]:
        """The work lists (parts.base.WorkList) that the blocks' parts want built for every step."""
        lists: Tuple[Any, ...] = ()
        for block in self.blocks:
            if hasattr(block, "work_lists"):
                lists += tuple(block.work_lists())
        return tuple(dict.fromkeys(lists))

    def decode_copy_bytes(self) -> Tuple[int, int]:
        """(bytes the decode copies of all parts take at most, bytes of the largest of them):
        every matrix of the checkpoint once more in the engine dtype; nothing for an engine
        dtype the decode kernels keep no copies for."""
        if self.dtype != torch.bfloat16:
            return 0, 0
        sizes = [2 * _numel(src.shape) for _, src in self.expected_tensors().values()
                 if src.kind == "matrix"]
        return sum(sizes), max(sizes, default=0)

    def widest_step_row_bytes(self) -> int:
        """Bytes of intermediate results one token of a step leaves in the widest block at most
        (every matrix product's output row, in the engine dtype, twice over for the
        element-wise results between them): what a recorded step's memory pool is sized by."""
        size = 4 if self.dtype == torch.float32 else 2
        widest = 0
        for block in self.blocks:
            parts = block.children().values() if hasattr(block, "children") else [block]
            rows = sum(src.shape[0] for p in parts for src in p.param_sources() if src.kind == "matrix")
            widest = max(widest, rows)
        return 2 * widest * size

    def graph_capturable(self) -> bool:
        """Whether a step of this model can be recorded as a HIP graph: every part says so."""
        return all(getattr(p, "graph_capturable", True)
                   for p in [self.embedding, *self.blocks, self.final_norm, self.head])

    @property
    def vocab_size(self) -> int:
        return self.head.vocab_size

    # ---- the forward pass of one step ------------------------------------------
    def forward(self, ctx, storage) -> torch.Tensor:
        """Float32 logits [len(ctx.logit_rows), vocab] for the flat batch ``ctx``."""
        h = self.embedding.forward(ctx.token_ids)
        residual = None
        last = len(self.schedule) - 1
        for i, call in enumerate(self.schedule):
            cache = storage.view(call.cache_layer, call.writes)
            block = self.blocks[call.block]
            # a block may leave its last product to the norm that comes next, if that norm can
            # take it (parts/base.py); the rows for the final norm are picked first, so not there
            after = self.blocks[self.schedule[i + 1].block] if i < last else None
            if (after is not None and getattr(block, "can_defer_output", False)
                    and getattr(after, "takes_pending_product", False)):
                h, residual = block.forward(h, residual, ctx, cache, defer_output=True)
            else:
                h, residual = block.forward(h, residual, ctx, cache)
        h = as_tensor(h)
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=h.device)
        if ctx.num_logit_rows != h.shape[0] or not ctx.logit_rows_are_identity:
            h = h.index_select(0, ctx.logit_rows)
            if residual is not None:
                residual = residual.index_select(0, ctx.logit_rows)
        h, _ = run_norm(self.final_norm, h, residual)
        return self.head.forward(as_tensor(h))
