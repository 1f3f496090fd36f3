"""Requests and their sampling parameters."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional

import numpy as np


@dataclass
class SamplingParams:
    """temperature 0 is greedy; otherwise softmax(logits/temperature) with
    nucleus top_p, as in the reference (temperature=0.6, top_p=0.9 are its
    defaults, lite_llama/generate_stream.py:91-99,143-150; max_gen_len there is
    max_new_tokens here)."""
    temperature: float = 0.6
    top_p: float = 0.9
    max_new_tokens: int = 128
    seed: Optional[int] = None        # None: derived from the engine seed and the request id
    ignore_eos: bool = False
    logprobs: bool = False            # report log_softmax(logits)[token] of every generated token

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")


WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass(eq=False)          # a request is itself: compared and hashed by identity
class Request:
    id: Hashable
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    output_logprobs: List[float] = field(default_factory=list)
    num_computed: int = 0             # tokens of prompt+output whose keys are in the cache
    status: str = WAITING
    finish_reason: Optional[str] = None
    num_preemptions: int = 0

    def __post_init__(self):
        # the prompt as a list and as an array: portions of it go to the step without a conversion
        self.prompt_array = np.asarray(self.prompt, dtype=np.int32).reshape(-1)
        if not isinstance(self.prompt, list):
            self.prompt = self.prompt_array.tolist()

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    def token_slice(self, start: int, n: int):
        """tokens[start:start+n] without joining prompt and output (a portion of the prompt
        as an int32 array, anything else as a list)."""
        np_ = len(self.prompt)
        if start + n <= np_:
            return self.prompt_array[start:start + n] if n > 1 else self.prompt[start:start + n]
        if start >= np_:
            return self.output[start - np_:start - np_ + n]
        return self.prompt[start:] + self.output[:start + n - np_]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def remaining(self) -> int:
        """Tokens not yet run through the model."""
        return self.num_tokens - self.num_computed


@dataclass
class StepOutput:
    request: Hashable
    token: int
    finished: bool
    finish_reason: Optional[str] = None
    logprob: Optional[float] = None
