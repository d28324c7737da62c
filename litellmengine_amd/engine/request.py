"""A request's life: waiting -> running -> finished.

Follows GenerationRequest / RequestManager of the reference
(include/engine/request.hpp:17-106, src/engine/request_manager.cpp:9-279):
`tokens` is prompt + generated (`input_ids` there), `cached_len` counts the
tokens whose K/V lie in the cache, the last sampled token is not yet cached
(`extend_len` = 1 while decoding), EOS is appended and then finishes the
request (:140-148), `max_new_tokens` reached finishes it (:150-155),
`max_new_tokens == 0` is finished at once (:30-34).
"""
from __future__ import annotations

import dataclasses
import enum
import random
from typing import List, Optional


class RequestStatus(enum.Enum):
    WAITING = "waiting"  # no cache slot (new, or preempted and to be recomputed)
    RUNNING = "running"  # holds a slot; prompt portions or decoding
    FINISHED = "finished"


@dataclasses.dataclass
class Request:
    request_id: int
    tokens: List[int]
    prompt_len: int
    max_new_tokens: int
    eos_token_id: int = -1
    temperature: float = 0.0
    seed: int = 0
    generated: List[int] = dataclasses.field(default_factory=list)
    cached_len: int = 0
    slot: int = -1
    status: RequestStatus = RequestStatus.WAITING
    admitted_at: int = -1  # order of admission; the youngest is preempted first
    preemptions: int = 0
    # a session: when it finishes it keeps its slot and pages, so that more input can be
    # appended and only the new tokens are run (finishing does not free in the reference,
    # src/engine/paged_generate_engine.cpp:386-395)
    keep_session: bool = False
    # 1 while a token has been picked for the request on the device and the host has not read it
    # yet (a step launched ahead): it counts as a token that is there but not cached
    pending: int = 0

    def __post_init__(self):
        # a stream of its own: what a request draws does not depend on its batch mates
        self.rng = random.Random((self.seed << 20) ^ (self.request_id * 0x9E3779B1))

    @property
    def device_len(self) -> int:
        return len(self.tokens)

    @property
    def extend_len(self) -> int:
        """Tokens not yet in the cache (include/engine/request.hpp:59-61)."""
        return len(self.tokens) + self.pending - self.cached_len

    @property
    def awaits_last_token(self) -> bool:
        """The token on its way is the last one the request may generate: nothing more to run."""
        return self.pending > 0 and len(self.generated) + self.pending >= self.max_new_tokens

    @property
    def remain_len(self) -> int:
        return self.prompt_len + self.max_new_tokens - len(self.tokens)

    @property
    def finished(self) -> bool:
        return self.status is RequestStatus.FINISHED

    def mark_forward_done(self, num_tokens: int) -> None:
        """src/engine/request_manager.cpp:190-213"""
        if num_tokens < 0 or self.cached_len + num_tokens > len(self.tokens) + self.pending:
            raise ValueError("mark_forward_done exceeds the request's tokens")
        self.cached_len += num_tokens

    def append_input_tokens(self, token_ids, max_new_tokens: int, eos_token_id: int) -> None:
        """A further turn: the history stays, the new tokens follow it, and what was
        generated before no longer counts against max_new_tokens
        (src/engine/request_manager.cpp:222-247, :256-279).  `cached_len` is left as
        it is: the new tokens reach the cache in the next steps."""
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        self.tokens.extend(int(t) for t in token_ids)
        self.generated = []
        self.prompt_len = len(self.tokens)
        self.max_new_tokens = max_new_tokens
        self.eos_token_id = int(eos_token_id)

    def append_token(self, token: int) -> None:
        """src/engine/request_manager.cpp:124-158"""
        if self.status is not RequestStatus.RUNNING:
            raise RuntimeError("append_token expects a running request")
        self.tokens.append(int(token))
        self.generated.append(int(token))
        if self.eos_token_id >= 0 and token == self.eos_token_id:
            self.status = RequestStatus.FINISHED
        elif len(self.generated) >= self.max_new_tokens:
            self.status = RequestStatus.FINISHED
