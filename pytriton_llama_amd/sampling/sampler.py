"""Choosing the next token of every request of a step."""
from __future__ import annotations

import hashlib
import struct
from typing import List, Optional, Sequence

import torch

from .. import ops
from ..engine.request import Request


def uniform_for(seed: int, request_seed, step: int) -> float:
    """A number in [0, 1) that depends only on (engine seed, request seed, index
    of the generated token): the same request draws the same numbers whatever
    else is in the batch and however its prompt was cut."""
    h = hashlib.blake2b(f"{seed}/{request_seed}/{step}".encode(), digest_size=8).digest()
    return (struct.unpack("<Q", h)[0] >> 11) * (1.0 / (1 << 53))


class Sampler:
    """Greedy rows take the arg-max kernel, the others the temperature / top-p
    kernel (the reference: logits/temperature, split softmax, sample_top_p with
    torch's global generator, or argmax when temperature is 0,
    lite_llama/generate_stream.py:143-150, lite_llama/generate.py:16-45)."""

    def __init__(self, seed: int = 0):
        self.seed = int(seed)
        self._wrote_host = False

    def logprobs_device(self, logits: torch.Tensor, requests: Sequence[Request],
                        tokens: torch.Tensor):
        """(indices of the requests that ask for log-probabilities, float32 device tensor of
        log_softmax(logits)[token] for them), from the unscaled logits as the reference does
        (lite_llama/generete_with_probs.py:154-165); (empty, None) when nobody asks."""
        want = [i for i, r in enumerate(requests) if r.params.logprobs]
        if not want:
            return want, None
        if len(want) == len(requests):
            rows, toks = logits, tokens
        else:
            idx = ops.to_device(want, torch.int32, logits.device)
            rows, toks = logits.index_select(0, idx), tokens.index_select(0, idx)
        return want, ops.token_logprob(rows, toks.contiguous())

    def logprobs(self, logits: torch.Tensor, requests: Sequence[Request], tokens: Sequence[int]):
        """As ``logprobs_device`` for tokens on the host: a list with None for the requests that
        do not ask."""
        out = [None] * len(requests)
        toks = ops.to_device(list(tokens), torch.int32, logits.device)
        want, lp = self.logprobs_device(logits, requests, toks)
        if want:
            for i, v in zip(want, lp.tolist()):
                out[i] = v
        return out

    def sample_device(self, logits: torch.Tensor, requests: Sequence[Request], ahead: int = 0,
                      host_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """logits float32 [R, V], row i for requests[i]; R token ids, int32, on the device (no
        wait for them). ``ahead``: how many tokens of each request are still on their way and
        not in its output list yet (they count for the index of the random number).
        ``host_out``: pinned int32 host memory that receives the tokens too (when every row is
        greedy the arg-max kernel writes them there itself, otherwise a copy is queued); it
        holds them once the work queued here has ended."""
        tokens = self._sample_device(logits, requests, ahead, host_out)
        if host_out is not None and tokens is not None and not self._wrote_host:
            host_out[:len(requests)].copy_(tokens, non_blocking=True)
        return tokens

    def _sample_device(self, logits, requests, ahead, host_out):
        self._wrote_host = False
        R = len(requests)
        if logits.shape[0] != R:
            raise ValueError(f"{logits.shape[0]} rows of logits for {R} requests")
        if R == 0:
            self._wrote_host = True
            return torch.empty((0,), dtype=torch.int32, device=logits.device)
        greedy = [i for i, r in enumerate(requests) if r.params.temperature == 0]
        if len(greedy) == R:
            self._wrote_host = host_out is not None
            return ops.argmax(logits, host_out)
        drawn = [i for i, r in enumerate(requests) if r.params.temperature != 0]
        params = []
        for i in drawn:
            r = requests[i]
            rs = r.params.seed if r.params.seed is not None else r.id
            params.append((r.params.temperature, r.params.top_p,
                           uniform_for(self.seed, rs, len(r.output) + ahead)))
        # (through pinned memory, without waiting: the step whose logits these are may still run)
        p = ops.to_device(list(zip(*params)), torch.float32, logits.device)
        if len(drawn) == R:
            return ops.sample_top_p(logits, p[0], p[1], p[2])
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        rows = ops.to_device(greedy + drawn, torch.int64, logits.device)
        gi, di = rows[:len(greedy)], rows[len(greedy):]
        out.index_copy_(0, gi, ops.argmax(logits.index_select(0, gi)))
        out.index_copy_(0, di, ops.sample_top_p(logits.index_select(0, di), p[0], p[1], p[2]))
        return out

    def sample(self, logits: torch.Tensor, requests: Sequence[Request]) -> List[int]:
        """As ``sample_device``, waited for: a list of R token ids."""
        return self.sample_device(logits, requests).tolist()
