"""A request as the scheduler sees it (src/engine/sequence.hpp:8-32): its tokens, prompt then
generated, its status, and what it holds in the cache."""
from __future__ import annotations

import enum
from typing import List, Optional

from ..cache.manager import RequestCache
from ..sampling.sampler import SamplingParams


class SequenceStatus(enum.Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


class Sequence:
    def __init__(self, seq_id: int, prompt_tokens: List[int], params: SamplingParams):
        self.id = seq_id
        self.status = SequenceStatus.WAITING
        self.tokens: List[int] = list(prompt_tokens)
        self.num_prompt_tokens = len(self.tokens)
        self.params = params
        self.cache: Optional[RequestCache] = None
        self.finish_reason: Optional[str] = None
        self.num_preemptions = 0
        #: draws of the sampler made in earlier turns of this request (a further turn goes on in the same stream of
        #: uniform numbers instead of starting it again)
        self.draws_before = 0
        self.admit_order = -1

    def __len__(self) -> int:
        return len(self.tokens)

    @property
    def num_computed(self) -> int:
        """Tokens whose keys and values are in the cache."""
        return self.cache.num_tokens if self.cache is not None else 0

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.num_prompt_tokens

    @property
    def num_draws(self) -> int:
        """Index of the request's next draw of the sampler."""
        return self.draws_before + self.num_generated

    @property
    def is_prefill(self) -> bool:
        """More than the last token is still to be computed."""
        return len(self.tokens) - self.num_computed > 1
