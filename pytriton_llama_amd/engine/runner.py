"""The step function: run a batch of (request, next tokens) through the model
from the cache and return the logits at the wanted places."""
from __future__ import annotations

from typing import Hashable, List, Optional, Sequence

import torch

from .. import ops
from ..cache import CacheManager, CacheStorage
from .batch import StepEntry, build_context


class ModelRunner:
    """Owns the cache (bookkeeping and device memory) of one loaded model.

    ``step`` runs only the tokens it is given, as one batch: portions of
    prompts beside single decoded tokens, cut anywhere. A request is admitted
    when it first appears and lives until ``end``. The reference's counterpart
    is ModelExecutor.forward with prefill_alloc_kv_cache / decode_alloc_kv_cache
    around it (lite_llama/executor/model_executor.py:261-320)."""

    def __init__(self, model, page_size: int, num_pages, max_num_seqs: int,
                 max_model_len: Optional[int] = None, use_graphs: bool = False,
                 timed_library_products: bool = True):
        if model.dtype is None:
            raise RuntimeError("load the model's weights before making a runner")
        self.model = model
        self.device = model.device
        if self.device.type == "cuda":
            ops.library.require(model.kernel_libraries())
        self.manager = CacheManager(model.cache_layers, page_size, num_pages, max_num_seqs)
        self.storage = CacheStorage(self.manager, model.dtype, self.device)
        # decode-only steps replay a HIP graph when the longest request is known
        self.graphs = None
        self.portion_graphs = None
        if (use_graphs and max_model_len and self.device.type == "cuda"
                and model.graph_capturable()):
            from .graphs import DecodeGraphs, PortionGraphs
            pool = torch.cuda.graph_pool_handle()
            self.graphs = DecodeGraphs(model, self.manager, self.storage, max_model_len, self.device,
                                       pool, timed_library_products)
            self.portion_graphs = PortionGraphs(model, self.manager, self.storage, max_model_len,
                                                self.device, pool, timed_library_products)

    def admit(self, request: Hashable) -> None:
        slot = self.manager.admit(request)
        self.storage.clear_slot(slot)

    @torch.inference_mode()
    def replays(self, entries: Sequence[StepEntry]) -> bool:
        """Whether this step would run as a captured graph (all entries decode one token)."""
        return self.graphs is not None and self.graphs.fits(entries)

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], token_feed=None) -> torch.Tensor:
        """Float32 logits [wanted, vocab], in the order of the entries and of
        their ``want`` lists. With graphs on, the result of a decode-only step is the graph's
        own buffer: it holds until the next step of this runner (work queued on the same
        stream before that step reads it safely; copy what has to last longer). ``token_feed``: the entries' tokens as an int32 device tensor,
        for a step that replays a graph and is launched before the host knows its tokens."""
        for e in entries:
            if not self.manager.is_live(e.request):
                self.admit(e.request)
        if self.graphs is not None and self.graphs.fits(entries):
            logits = self.graphs.step(entries, token_feed)
        elif token_feed is not None:
            raise ValueError("only steps that replay a graph can take their tokens from the device")
        elif self.portion_graphs is not None and self.portion_graphs.fits(entries):
            logits = self.portion_graphs.step(entries)
        else:
            ctx, _ = build_context(entries, self.manager, self.device, self.model.vocab_size,
                                   self.model.work_lists())
            logits = self.model.forward(ctx, self.storage)
        for e in entries:
            self.manager.release_behind_window(e.request)
        return logits

    def end(self, request: Hashable) -> None:
        """The request is finished: what it holds is given back."""
        if self.manager.is_live(request):
            self.manager.free(request)
