"""Continuous batching for the ragged stack engine: which tokens of which requests the next step carries.

The engine takes packed steps - portions of prompts next to single decoded tokens - so the scheduler's whole job is to fill a
token budget per step: every running request that is decoding contributes its last sampled token, the rest of the budget goes to
prompts (running ones first, then newly admitted ones), cut wherever the budget ends.  A request is admitted when a state slot is
free and the block pool can hold its prompt plus everything it may generate, so nothing is ever pre-empted."""
import collections
from dataclasses import dataclass, field
from typing import List, Optional, Tuple


@dataclass
class Request:
    rid: object
    prompt: List[int]
    max_new_tokens: int
    end_id: Optional[int] = None
    fed: int = 0                     # tokens of prompt + output that have been run
    output: List[int] = field(default_factory=list)
    finished: bool = False

    def tokens(self) -> List[int]:
        return list(self.prompt) + self.output

    def pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.fed


class RaggedScheduler(object):

    def __init__(self, max_batch_tokens: int, max_sequences: int, page_size: int, num_blocks: int):
        if max_batch_tokens < 1 or max_sequences < 1:
            raise ValueError('max_batch_tokens and max_sequences must be positive')
        self.max_batch_tokens, self.max_sequences = max_batch_tokens, max_sequences
        self.page_size, self.num_blocks = page_size, num_blocks
        self.waiting = collections.deque()
        self.running: List[Request] = []
        self._committed = {}  # rid -> blocks promised to the request

    def _blocks_for(self, r: Request) -> int:
        return -(-(len(r.prompt) + r.max_new_tokens) // self.page_size)

    def add(self, r: Request):
        if not r.prompt:
            raise ValueError('empty prompt')
        if self._blocks_for(r) > self.num_blocks:
            raise ValueError(f'request {r.rid}: {len(r.prompt)} + {r.max_new_tokens} tokens do not fit the pool of '
                             f'{self.num_blocks} blocks of {self.page_size}')
        self.waiting.append(r)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def schedule(self) -> List[Tuple[Request, int]]:
        """[(request, tokens to run now)]: decoding requests first (one token each), then prompt portions."""
        budget = self.max_batch_tokens
        step = []
        for r in self.running:
            if r.output and r.pending() == 1 and budget > 0:
                step.append((r, 1))
                budget -= 1
        for r in self.running:
            if not r.output and budget > 0:
                n = min(r.pending(), budget)
                step.append((r, n))
                budget -= n
        while self.waiting and budget > 0 and len(self.running) < self.max_sequences:
            r = self.waiting[0]
            need = self._blocks_for(r)
            if sum(self._committed.values()) + need > self.num_blocks:
                break
            self.waiting.popleft()
            self._committed[r.rid] = need
            self.running.append(r)
            n = min(r.pending(), budget)
            step.append((r, n))
            budget -= n
        return step

    def update(self, r: Request, ran: int, next_id: Optional[int]) -> bool:
        """After a step: `ran` tokens of r were run; next_id is the sampler's choice behind its last token when that token was the
        last one known (None for a prompt portion that ends before the prompt does).  True when r has finished."""
        r.fed += ran
        if next_id is not None and r.pending() == 0:
            r.output.append(int(next_id))
            if len(r.output) >= r.max_new_tokens or (r.end_id is not None and int(next_id) == r.end_id):
                r.finished = True
                self.running.remove(r)
                del self._committed[r.rid]
        return r.finished
