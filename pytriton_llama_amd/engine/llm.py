"""The engine: a loaded model, its runner, a scheduler and a sampler."""
from __future__ import annotations

import itertools
import os
from typing import Dict, Hashable, Iterator, List, Optional, Sequence, Union

import numpy as np
import torch

from ..cache import CacheManager, CacheStorage
from ..config import EngineConfig, build_model, read_config_json
from ..sampling import Sampler
from ..weights import load_random_weights, load_weights
from .batch import StepEntry
from .request import Request, SamplingParams, StepOutput
from .runner import ModelRunner
from .scheduler import Scheduler


def pages_that_fit(usable_bytes: int, bytes_per_page: int, state_bytes: int, cap: int) -> int:
    """Pages for ``usable_bytes`` of memory when the fixed-size state of all slots takes
    ``state_bytes`` of it first; at most ``cap``. A model without paged layers needs no page
    (one is kept so that the pools exist)."""
    left = usable_bytes - state_bytes
    if left < 0:
        raise RuntimeError(f"the fixed-size state of the requests ({state_bytes} bytes) does not fit "
                           f"into the {max(usable_bytes, 0)} bytes left after loading the weights")
    if bytes_per_page <= 0:
        return 1
    n = min(left // bytes_per_page, cap)
    if n < 1:
        raise RuntimeError("no memory left for the cache after loading the weights")
    return int(n)


def graph_pool_bytes(model, engine: EngineConfig) -> int:
    """Memory the recorded steps' shared pool is allowed for when the cache is sized from free
    memory: the intermediate results of the largest step that is recorded (a portion of up to
    2,048 tokens beside max_num_seqs decoding rows) and its float32 logits. Nothing when steps
    are not recorded."""
    if not (engine.use_graphs and model.graph_capturable()):
        return 0
    from .graphs import PORTION_BUCKETS
    tokens = min(PORTION_BUCKETS[-1], engine.max_num_batched_tokens) + engine.max_num_seqs
    return tokens * model.widest_step_row_bytes() + (engine.max_num_seqs + 1) * model.vocab_size * 4


def pages_from_memory(model, engine: EngineConfig) -> int:
    """Pages that fit into gpu_memory_fraction of the device after the weights
    are loaded (the reference: (total*0.9 - peak - non_torch) // bytes per block,
    lite_llama/executor/mem_manager.py:44-60,98-110), less what the state pools and the
    recorded steps' memory pool take."""
    probe = CacheManager(model.cache_layers, engine.page_size, 1, engine.max_num_seqs)
    per_page = CacheStorage.bytes_per_page(probe, engine.dtype)
    fixed = CacheStorage.state_bytes(probe, engine.dtype) + graph_pool_bytes(model, engine)
    free, total = torch.cuda.mem_get_info(torch.device(engine.device))
    usable = int(total * engine.gpu_memory_fraction) - (total - free)
    # no request can use more than max_model_len, and max_num_seqs of them may live
    cap = engine.max_num_seqs * (-(-engine.max_model_len // engine.page_size))
    return pages_that_fit(usable, per_page, fixed, cap)


def decode_copies_fit(copies_bytes: int, largest_copy_bytes: int, free_bytes: int,
                      keep_free_bytes: int) -> bool:
    """Whether the second copies of the weights for decode steps may be made: they take
    ``copies_bytes`` for good and, while one is built, its size once more; ``keep_free_bytes``
    must remain for the cache."""
    return copies_bytes + largest_copy_bytes + keep_free_bytes <= free_bytes


def make_decode_copies_if_room(model, device, keep_free_bytes: int) -> bool:
    """Build the parts' decode copies unless they would not leave ``keep_free_bytes`` of device
    memory; says so on stderr when it leaves them out (the model then runs its decode steps
    from the row-major weights, somewhat slower)."""
    copies, largest = model.decode_copy_bytes()
    free, _ = torch.cuda.mem_get_info(torch.device(device))
    if not decode_copies_fit(copies, largest, free, keep_free_bytes):
        import sys
        print(f"[pytriton_llama_amd] no second copies of the weights for decode steps: they need "
              f"{(copies + largest) >> 20} MiB beside {keep_free_bytes >> 20} MiB for the cache, "
              f"{free >> 20} MiB are free (decode_weight_copies=False says the same without trying)",
              file=sys.stderr, flush=True)
        return False
    model.make_decode_copies()
    return True


def cache_floor_bytes(model, engine: EngineConfig) -> int:
    """The least the cache must get: the pages the engine was told to have, or those of one
    request of max_model_len tokens, plus the state pools and the recorded steps' pool."""
    probe = CacheManager(model.cache_layers, engine.page_size, 1, engine.max_num_seqs)
    pages = engine.num_pages if engine.num_pages is not None else -(-engine.max_model_len // engine.page_size)
    return (pages * CacheStorage.bytes_per_page(probe, engine.dtype)
            + CacheStorage.state_bytes(probe, engine.dtype) + graph_pool_bytes(model, engine))


class _Launched:
    """A step that is under way: its plan, the requests that get a token from it (in the order
    of the token tensors), the tokens on the device and the pinned buffers they are copied to,
    the event after those copies."""
    __slots__ = ("plan", "samplers", "tokens", "host_tokens", "want_lp", "host_lps", "done",
                 "replayed")

    def __init__(self, plan, samplers, tokens, host_tokens, want_lp, host_lps, done, replayed):
        self.plan, self.samplers, self.tokens = plan, samplers, tokens
        self.host_tokens, self.want_lp, self.host_lps = host_tokens, want_lp, host_lps
        self.done, self.replayed = done, replayed


class Engine:
    """Model folder (or a config dict with ``random_seed``, or a model that is built and loaded)
    -> generated tokens.

        engine = Engine("/path/to/model", EngineConfig(dtype="bfloat16"))
        outs = engine.generate([[1, 2, 3]], SamplingParams(temperature=0, max_new_tokens=8))
    """

    def __init__(self, model: Union[str, dict], engine_config: Optional[EngineConfig] = None,
                 random_seed: Optional[int] = None, norm_std: float = 0.0, weight_std=None):
        self.config = engine_config or EngineConfig()
        ec = self.config
        if torch.device(ec.device).type != "cuda":
            raise RuntimeError("the engine runs on a GPU only; there is no CPU path")
        if hasattr(model, "schedule") and hasattr(model, "blocks"):
            # a model that is built and loaded (a CausalLM): another engine may share its weights
            if model.dtype != ec.dtype or str(model.device) != str(torch.device(ec.device)):
                raise ValueError(f"the model holds {model.dtype} on {model.device}, the engine is "
                                 f"configured for {ec.dtype} on {ec.device}")
            self.model = model
        elif isinstance(model, str):
            cfg = read_config_json(model)
            self.model = build_model(cfg)
            if random_seed is None:
                load_weights(self.model, model, ec.dtype, ec.device)
            else:
                load_random_weights(self.model, random_seed, ec.dtype, ec.device, norm_std, weight_std)
        else:
            self.model = build_model(model)
            load_random_weights(self.model, random_seed or 0, ec.dtype, ec.device, norm_std, weight_std)
        if ec.decode_weight_copies and not self.model.has_decode_copies:
            make_decode_copies_if_room(self.model, ec.device, cache_floor_bytes(self.model, ec))
        num_pages = ec.num_pages if ec.num_pages is not None else pages_from_memory(self.model, ec)
        self.runner = ModelRunner(self.model, ec.page_size, num_pages, ec.max_num_seqs,
                                  ec.max_model_len, ec.use_graphs, ec.timed_library_products)
        eos = getattr(self.model.config, "eos_token_ids", ())
        self.scheduler = Scheduler(self.runner.manager, ec.max_num_seqs, ec.max_num_batched_tokens,
                                   ec.prefill_chunk, ec.max_model_len, eos)
        self.sampler = Sampler(ec.seed)
        self.requests: Dict[Hashable, Request] = {}
        self._ids = itertools.count()
        # a step that has been launched and whose tokens have not been fetched yet; pinned
        # buffers for the fetches, used in turn (two steps are under way at most)
        self._inflight: Optional[_Launched] = None
        self._pinned = [(torch.empty(ec.max_num_seqs, dtype=torch.int32).pin_memory(),
                         torch.empty(ec.max_num_seqs, dtype=torch.float32).pin_memory())
                        for _ in range(3)]
        self._turn = 0

    # ---- requests ------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None) -> Hashable:
        rid = request_id if request_id is not None else next(self._ids)
        if rid in self.requests:
            raise ValueError(f"request id {rid!r} is in use")
        V = self.model.vocab_size
        ids = np.asarray(prompt if not isinstance(prompt, torch.Tensor) else prompt.cpu())
        if ids.ndim != 1 or (ids.size and ids.dtype.kind not in "iu"):
            raise ValueError("a prompt is a sequence of token ids (integers)")
        outside = ids[(ids < 0) | (ids >= V)]
        if outside.size:
            raise ValueError(f"token id {int(outside[0])} outside the vocabulary of {V}")
        req = Request(rid, ids.astype(np.int32), params or SamplingParams())
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    def step(self) -> List[StepOutput]:
        """One step of the whole engine: plan, run, sample, record. While every running
        request decodes (and ``async_decode`` is on), the step after this one is launched
        before this one's tokens are fetched: its tokens travel from the sampler to the model
        on the device, and the host's planning and book-keeping run beside the GPU's work.
        Each call still returns the tokens of exactly one step, in order."""
        if self._inflight is None:
            self._inflight = self._launch(self.scheduler.schedule(), None)
        cur, nxt = self._inflight, None
        if self.config.async_decode and cur.replayed:
            ahead = self.scheduler.plan_ahead(cur.plan)
            if ahead is not None:
                nxt = self._launch(ahead, cur)
        outs = self._collect(cur)
        self._inflight = nxt
        return outs

    def _launch(self, plan, before: Optional["_Launched"]) -> "_Launched":
        """Start the step ``plan`` and the sampling of its tokens; nothing is waited for.
        ``before``: the step whose tokens this one consumes while they are still on the device
        (same requests in the same order, one token each)."""
        entries, samplers = [], []
        for e in plan.entries:
            toks = [0] if before is not None else e.request.token_slice(e.start, e.num_tokens)
            entries.append(StepEntry(e.request.id, toks, [e.num_tokens - 1] if e.samples else []))
            if e.samples:
                samplers.append(e.request)
        replayed = self.runner.replays(entries)
        logits = self.runner.step(entries, before.tokens if before is not None else None)
        ahead = 1 if before is not None else 0
        host_tokens, host_lps = self._pinned[self._turn % len(self._pinned)]
        self._turn += 1
        tokens = self.sampler.sample_device(logits, samplers, ahead, host_tokens)
        want_lp, lps = self.sampler.logprobs_device(logits, samplers, tokens)
        if want_lp:
            host_lps[:len(want_lp)].copy_(lps, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return _Launched(plan, samplers, tokens, host_tokens, want_lp, host_lps, done, replayed)

    def _collect(self, step: "_Launched") -> List[StepOutput]:
        """Wait for the step's tokens and record them."""
        step.done.synchronize()
        n = len(step.samplers)
        tokens = step.host_tokens[:n].tolist()
        outs = self.scheduler.update(step.plan, {r.id: t for r, t in zip(step.samplers, tokens)})
        if step.want_lp:
            lps = step.host_lps[:len(step.want_lp)].tolist()
            by_id = {step.samplers[i].id: lp for i, lp in zip(step.want_lp, lps)}
            for o in outs:
                if o.request in by_id:
                    o.logprob = by_id[o.request]
                    self.requests[o.request].output_logprobs.append(o.logprob)
        return outs

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work or self._inflight is not None

    def abort(self, request_id: Hashable) -> None:
        """Stop a request: what it holds is given back; a step that is under way still
        finishes, and what it computed for this request is dropped."""
        req = self.requests.pop(request_id, None)
        if req is not None:
            self.scheduler.abort(req)
        if self._inflight is not None and not self.scheduler.has_work:
            self._collect(self._inflight)
            self._inflight = None

    def warm_up(self, decode_batches: Optional[Sequence[int]] = None,
                portion_sizes: Optional[Sequence[int]] = None) -> None:
        """Capture the HIP graphs before the first request needs them (a capture takes about
        0.1 s): decode steps of the given batch sizes (default: every bucket) and steps with
        one prompt portion of the given sizes alone (default: every bucket that the token
        budget and ``max_model_len`` allow). Only on an idle engine; the requests it makes up
        are gone when it returns."""
        if self.has_work:
            raise RuntimeError("warm_up needs an idle engine")
        runner = self.runner
        if runner.graphs is None:
            return
        from .batch import StepEntry
        limit = min(self.config.max_num_batched_tokens, self.config.max_model_len)
        if portion_sizes is None:
            portion_sizes = [t for t in runner.portion_graphs.sizes if t <= limit]
        if decode_batches is None:
            decode_batches = runner.graphs.sizes
        for t in portion_sizes:
            if self.manager_fits(t, 1):
                runner.step([StepEntry(("warm-up", t), [0] * t, [t - 1])])
                runner.end(("warm-up", t))
        for b in decode_batches:
            if b <= self.config.max_num_seqs and self.manager_fits(1, b):
                names = [("warm-up", b, i) for i in range(b)]
                runner.step([StepEntry(n, [0], [0]) for n in names])
                for n in names:
                    runner.end(n)
        torch.cuda.synchronize()

    def manager_fits(self, tokens_each: int, requests: int) -> bool:
        """Whether the free pages hold ``requests`` new requests of ``tokens_each`` tokens."""
        m = self.runner.manager
        pages = -(-tokens_each // m.page_size) * requests
        return all(g.pool.num_free >= pages for g in m.paged)

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
