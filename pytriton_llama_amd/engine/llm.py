"""The engine: a loaded model, its runner, a scheduler and a sampler."""
from __future__ import annotations

import itertools
import os
from typing import Dict, Hashable, Iterator, List, Optional, Sequence, Union

import torch

from ..cache import CacheManager, CacheStorage
from ..config import EngineConfig, build_model, read_config_json
from ..sampling import Sampler
from ..weights import load_random_weights, load_weights
from .batch import StepEntry
from .request import Request, SamplingParams, StepOutput
from .runner import ModelRunner
from .scheduler import Scheduler


def pages_from_memory(model, engine: EngineConfig) -> int:
    """Pages that fit into gpu_memory_fraction of the device after the weights
    are loaded (the reference: (total*0.9 - peak - non_torch) // bytes per block,
    lite_llama/executor/mem_manager.py:44-60,98-110)."""
    probe = CacheManager(model.cache_layers, engine.page_size, 1, engine.max_num_seqs)
    per_page = CacheStorage.bytes_per_page(probe, engine.dtype)
    free, total = torch.cuda.mem_get_info(torch.device(engine.device))
    usable = int(total * engine.gpu_memory_fraction) - (total - free)
    # no request can use more than max_model_len, and max_num_seqs of them may live
    cap = engine.max_num_seqs * (-(-engine.max_model_len // engine.page_size))
    n = min(max(usable // max(per_page, 1), 0), cap)
    if n < 1:
        raise RuntimeError("no memory left for the cache after loading the weights")
    return n


class Engine:
    """Model folder (or a config dict with ``random_seed``) -> generated tokens.

        engine = Engine("/path/to/model", EngineConfig(dtype="bfloat16"))
        outs = engine.generate([[1, 2, 3]], SamplingParams(temperature=0, max_new_tokens=8))
    """

    def __init__(self, model: Union[str, dict], engine_config: Optional[EngineConfig] = None,
                 random_seed: Optional[int] = None, norm_std: float = 0.0, weight_std=None):
        self.config = engine_config or EngineConfig()
        ec = self.config
        if torch.device(ec.device).type != "cuda":
            raise RuntimeError("the engine runs on a GPU only; there is no CPU path")
        if isinstance(model, str):
            cfg = read_config_json(model)
            self.model = build_model(cfg)
            if random_seed is None:
                load_weights(self.model, model, ec.dtype, ec.device)
            else:
                load_random_weights(self.model, random_seed, ec.dtype, ec.device, norm_std, weight_std)
        else:
            self.model = build_model(model)
            load_random_weights(self.model, random_seed or 0, ec.dtype, ec.device, norm_std, weight_std)
        num_pages = ec.num_pages if ec.num_pages is not None else pages_from_memory(self.model, ec)
        self.runner = ModelRunner(self.model, ec.page_size, num_pages, ec.max_num_seqs,
                                  ec.max_model_len, ec.use_graphs)
        eos = getattr(self.model.config, "eos_token_ids", ())
        self.scheduler = Scheduler(self.runner.manager, ec.max_num_seqs, ec.max_num_batched_tokens,
                                   ec.prefill_chunk, ec.max_model_len, eos)
        self.sampler = Sampler(ec.seed)
        self.requests: Dict[Hashable, Request] = {}
        self._ids = itertools.count()

    # ---- requests ------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None) -> Hashable:
        rid = request_id if request_id is not None else next(self._ids)
        if rid in self.requests:
            raise ValueError(f"request id {rid!r} is in use")
        V = self.model.vocab_size
        for t in prompt:
            if not 0 <= int(t) < V:
                raise ValueError(f"token id {t} outside the vocabulary of {V}")
        req = Request(rid, [int(t) for t in prompt], params or SamplingParams())
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    def step(self) -> List[StepOutput]:
        """One step of the whole engine: plan, run, sample, record."""
        plan = self.scheduler.schedule()
        entries, samplers = [], []
        for e in plan.entries:
            toks = e.request.token_slice(e.start, e.num_tokens)
            entries.append(StepEntry(e.request.id, toks, [e.num_tokens - 1] if e.samples else []))
            if e.samples:
                samplers.append(e.request)
        logits = self.runner.step(entries)
        tokens = self.sampler.sample(logits, samplers)
        logprobs = self.sampler.logprobs(logits, samplers, tokens)
        outs = self.scheduler.update(plan, {r.id: t for r, t in zip(samplers, tokens)})
        by_id = {r.id: lp for r, lp in zip(samplers, logprobs) if lp is not None}
        for o in outs:
            if o.request in by_id:
                o.logprob = by_id[o.request]
                self.requests[o.request].output_logprobs.append(o.logprob)
        return outs

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work

    # ---- whole generations ----------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[List[int]]:
        """Generated token ids (without the prompt) for every prompt."""
        return [r.output for r in self.generate_requests(prompts, params)]

    def generate_requests(self, prompts, params=None) -> List[Request]:
        """As ``generate``, returning the finished requests (tokens, log-probabilities,
        finish reasons)."""
        ids = self._add_all(prompts, params)
        while self.has_work:
            self.step()
        return [self.requests.pop(i) for i in ids]

    def generate_stream(self, prompts, params=None) -> Iterator[List[StepOutput]]:
        """Yields, step by step, the new token of every request that got one;
        StepOutput.request is the index of the prompt."""
        ids = self._add_all(prompts, params)
        index = {rid: i for i, rid in enumerate(ids)}
        while self.has_work:
            outs = self.step()
            mine = [StepOutput(index[o.request], o.token, o.finished, o.finish_reason, o.logprob)
                    for o in outs if o.request in index]
            if mine:
                yield mine
        for rid in ids:
            self.requests.pop(rid, None)

    def _add_all(self, prompts, params):
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        return [self.add_request(p, sp) for p, sp in zip(prompts, params)]
