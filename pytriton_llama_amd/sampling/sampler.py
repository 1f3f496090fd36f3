"""Choosing the next token of every request of a step."""
from __future__ import annotations

import hashlib
import struct
from typing import List, Sequence

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

    def logprobs(self, logits: torch.Tensor, requests: Sequence[Request], tokens: Sequence[int]):
        """log_softmax(logits)[token] for the requests that ask for it (None for the others),
        from the unscaled logits as the reference does
        (lite_llama/generete_with_probs.py:154-165)."""
        want = [i for i, r in enumerate(requests) if r.params.logprobs]
        out = [None] * len(requests)
        if not want:
            return out
        rows = logits if len(want) == len(requests) else logits.index_select(
            0, torch.tensor(want, dtype=torch.int32, device=logits.device))
        toks = torch.tensor([tokens[i] for i in want], dtype=torch.int32, device=logits.device)
        for i, lp in zip(want, ops.token_logprob(rows, toks).tolist()):
            out[i] = lp
        return out

    def sample(self, logits: torch.Tensor, requests: Sequence[Request]) -> List[int]:
        """logits float32 [R, V], row i for requests[i]; returns R token ids."""
        R = len(requests)
        if logits.shape[0] != R:
            raise ValueError(f"{logits.shape[0]} rows of logits for {R} requests")
        if R == 0:
            return []
        greedy = [i for i, r in enumerate(requests) if r.params.temperature == 0]
        drawn = [i for i, r in enumerate(requests) if r.params.temperature != 0]
        out = [0] * R
        if len(greedy) == R:
            return ops.argmax(logits).tolist()
        if greedy:
            idx = torch.tensor(greedy, dtype=torch.int32, device=logits.device)
            for i, t in zip(greedy, ops.argmax(logits.index_select(0, idx)).tolist()):
                out[i] = t
        rows = logits if len(drawn) == R else logits.index_select(
            0, torch.tensor(drawn, dtype=torch.int32, device=logits.device))
        params = []
        for i in drawn:
            r = requests[i]
            rs = r.params.seed if r.params.seed is not None else r.id
            params.append((r.params.temperature, r.params.top_p,
                           uniform_for(self.seed, rs, len(r.output))))
        p = torch.tensor(params, dtype=torch.float32).t().contiguous().to(logits.device)
        for i, t in zip(drawn, ops.sample_top_p(rows, p[0], p[1], p[2]).tolist()):
            out[i] = t
        return out
