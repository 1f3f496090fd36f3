"""The Python entry points in the reference's manner: GenerateText and
GenerateStreamText with its names and meanings of options
(lite_llama/generate.py:47-206, lite_llama/generate_stream.py:51-216).

Differences that follow from the engine underneath: prompts of unequal length
are not padded (every request has its own positions), a finished request stops
computing, and a tokenizer is optional: without one the token-id methods work
and the text methods raise.
"""
from __future__ import annotations

import os
from typing import Generator, List, Optional, Sequence, Tuple

from .config import EngineConfig
from .engine import Engine, SamplingParams


def load_tokenizer(path: Optional[str]):
    """tokenizer.json of the model folder through the ``tokenizers`` package;
    None when there is none (the reference uses transformers.AutoTokenizer,
    lite_llama/generate.py:78-85)."""
    if not path:
        return None
    f = os.path.join(path, "tokenizer.json") if os.path.isdir(path) else path
    if not os.path.isfile(f):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(f)


class GenerateText:
    """checkpoints_dir: model folder (config.json + safetensors). max_seq_len
    caps prompt + generated tokens. max_gpu_num_blocks: size of the cache pool in
    pages (None: from free memory). load_model False starts from random weights
    (seeded) instead of reading the folder's tensors. triton_weight is accepted
    for compatibility (there is one weight format). compiled_model switches the
    replay of decode steps and of single prompt portions as HIP graphs, and with
    it the launch of a decode step ahead of the tokens of the step before; it is
    on by default (the reference's flag defaults to off, lite_llama/generate.py:59,
    and its captured graphs are never replayed, model_executor.py:314-320; here
    the replayed step is the fast path and the one that is measured)."""

    def __init__(self, checkpoints_dir: str, tokenizer_path: Optional[str] = None,
                 max_seq_len: int = 1024, max_gpu_num_blocks: Optional[int] = None,
                 load_model: bool = True, triton_weight: bool = True, compiled_model: bool = True,
                 device: str = "cuda", dtype: str = "bfloat16", seed: int = 0,
                 page_size: int = 16, max_batch_size: int = 64,
                 max_num_batched_tokens: int = 2048, prefill_chunk: Optional[int] = None):
        dev = "cuda:0" if device == "cuda" else device
        self.engine_config = EngineConfig(
            dtype=dtype, device=dev, page_size=page_size, num_pages=max_gpu_num_blocks,
            max_num_seqs=max_batch_size, max_num_batched_tokens=max_num_batched_tokens,
            prefill_chunk=prefill_chunk, max_model_len=max_seq_len, seed=seed,
            use_graphs=compiled_model)
        self.engine = Engine(checkpoints_dir, self.engine_config,
                             random_seed=None if load_model else seed)
        self.model_config = self.engine.model.config
        self.tokenizer = load_tokenizer(tokenizer_path or checkpoints_dir)

    def _params(self, max_gen_len, temperature, top_p, n_prompt, logprobs=False):
        room = self.engine_config.max_model_len - n_prompt
        if room < 1:
            raise ValueError(f"a prompt of {n_prompt} tokens leaves no room under max_seq_len "
                             f"{self.engine_config.max_model_len}")
        return SamplingParams(temperature=temperature, top_p=top_p,
                              max_new_tokens=max(1, min(max_gen_len, room)), logprobs=logprobs)

    def generate(self, prompt_tokens: List[List[int]], max_gen_len: int, temperature: float = 0.6,
                 top_p: float = 0.9, echo: bool = False, logprobs: bool = False
                 ) -> Tuple[List[List[int]], Optional[List[List[float]]]]:
        """Token ids generated for every prompt (with the prompt in front when
        ``echo``); generation of a request stops at its EOS token. With ``logprobs``
        the second result holds log_softmax(logits)[token] of every generated token
        (the reference's generete_with_probs.py:89-97,154-165; prompt tokens under
        ``echo`` have none and are not listed)."""
        params = [self._params(max_gen_len, temperature, top_p, len(p), logprobs) for p in prompt_tokens]
        reqs = self.engine.generate_requests(prompt_tokens, params)
        outs = [r.output for r in reqs]
        if echo:
            outs = [list(p) + o for p, o in zip(prompt_tokens, outs)]
        return outs, ([r.output_logprobs for r in reqs] if logprobs else None)

    def _need_tokenizer(self):
        if self.tokenizer is None:
            raise RuntimeError("no tokenizer.json in the model folder: use the token-id methods")

    def _encode(self, prompts: Sequence[str]) -> List[List[int]]:
        self._need_tokenizer()
        return [self.tokenizer.encode(x, add_special_tokens=True).ids for x in prompts]

    def text_completion(self, prompts: List[str], temperature: float = 0.6, top_p: float = 0.9,
                        max_gen_len: Optional[int] = None, echo: bool = False) -> List[dict]:
        if max_gen_len is None:
            max_gen_len = self.engine_config.max_model_len - 1
        toks, _ = self.generate(self._encode(prompts), max_gen_len, temperature, top_p, echo)
        eos = set(self.model_config.eos_token_ids)
        return [{"generation": self.tokenizer.decode([t for t in ts if t not in eos],
                                                     skip_special_tokens=True)} for ts in toks]


class GenerateStreamText(GenerateText):
    def generate_stream(self, prompt_tokens: List[List[int]], max_gen_len: int,
                        temperature: float = 0.6, top_p: float = 0.9, echo: bool = False
                        ) -> Generator[List[List[int]], None, None]:
        """Yields after every step, for every prompt, the token ids that are new
        since the last yield (the reference yields their text,
        lite_llama/generate_stream.py:169-182)."""
        params = [self._params(max_gen_len, temperature, top_p, len(p)) for p in prompt_tokens]
        first = True
        for outs in self.engine.generate_stream(prompt_tokens, params):
            batch = [[] for _ in prompt_tokens]
            if echo and first:
                batch = [list(p) for p in prompt_tokens]
            first = False
            for o in outs:
                batch[o.request].append(o.token)
            yield batch

    def text_completion_stream(self, prompts: List[str], temperature: float = 0.6,
                               top_p: float = 0.9, max_gen_len: Optional[int] = None,
                               echo: bool = False) -> Generator[List[dict], None, None]:
        if max_gen_len is None:
            max_gen_len = self.engine_config.max_model_len - 1
        eos = set(self.model_config.eos_token_ids)
        ids = [[] for _ in prompts]
        for batch in self.generate_stream(self._encode(prompts), max_gen_len, temperature, top_p, echo):
            for i, new in enumerate(batch):
                ids[i].extend(t for t in new if t not in eos)
            yield [{"generation": self.tokenizer.decode(ts, skip_special_tokens=True), "tokens": list(ts)}
                   for ts in ids]
