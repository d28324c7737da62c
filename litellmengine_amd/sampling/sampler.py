"""Picking the next token from float32 logits rows, on the GPU.

Greedy when a request's temperature is 0: first maximum wins
(src/ops/argmax.cu:49-59, :106-110).  Otherwise p = softmax(logits / T) in
float32 and an inverse-CDF draw with a uniform number from the request's own
generator, so that what a request draws does not depend on its batch mates.
The reference parses --temperature, --top-k and --top-p and then warns that
only greedy is implemented (src/main.cpp:175-178); top-k/top-p are accepted
and ignored here in the same way.
"""
from __future__ import annotations

from typing import List, Sequence

import torch


# the largest float32 below 1: a double just below 1 would round to 1.0 on its way to the kernel,
# where no id's share of the running sum reaches
MAX_UNIFORM = 1.0 - 2.0 ** -24


class Sampler:
    def __init__(self, ops, device):
        self.ops = ops
        self.device = device

    def pick(self, logits: torch.Tensor, requests: Sequence) -> List[int]:
        """logits [R, V] float32, one row per request (engine.request.Request)."""
        if logits.shape[0] != len(requests):
            raise ValueError("one logits row per sampling request")
        if logits.shape[0] == 0:
            return []
        if all(r.temperature <= 0.0 for r in requests):
            return self.ops.argmax(logits).tolist()
        temperature = [float(r.temperature) for r in requests]
        uniform = [min(r.rng.random(), MAX_UNIFORM) if r.temperature > 0.0 else 0.0 for r in requests]
        both = torch.tensor([temperature, uniform], dtype=torch.float32).to(self.device)
        return self.ops.sample(logits, both[0].contiguous(), both[1].contiguous()).tolist()
