"""Round-robin planner with a token budget, chunked prompts and admission between steps.

Policy of the reference's scheduler (qil/scheduler.py:37-103):
  * ``add`` refuses a request that could never fit the cache (:52-53).
  * ``plan`` first admits waiting requests while fewer than ``max_active`` are
    active and the cache can reserve their whole life (``len(prompt) +
    max_new_tokens - 1`` tokens: the last sampled token is never fed back,
    :24-27); a request that does not fit goes to the back of the queue, so a
    smaller later one may overtake it (:58-67).
  * then it hands out the step's token budget: at most one piece of work per
    active request, ``prefill_chunk`` tokens of a prompt or the one last sampled
    token of a decoding request, cut down to the remaining budget; served
    requests rotate to the back, so those left out come first next step (:68-84).
  * pages cannot run out inside a request, because admission reserved them; lack
    of room shows as waiting, or as refusal at ``add``.  Nothing is preempted,
    swapped or recomputed.
The plan is executed as one batch by the step function.
"""
from collections import deque
from dataclasses import dataclass, field


@dataclass
class Request:
    id: int
    prompt: list
    max_new_tokens: int
    eos: frozenset
    arrival_s: float
    temperature: float = 0.0
    seed: int = 0
    output: list = field(default_factory=list)
    token_times_s: list = field(default_factory=list)
    computed: int = 0
    state: str = 'waiting'               # waiting -> active -> completed | cancelled | failed
    finish_reason: str | None = None
    error: str | None = None

    @property
    def input_tokens(self):
        return self.prompt + self.output

    @property
    def cache_limit(self):
        return len(self.prompt) + self.max_new_tokens - 1


@dataclass(frozen=True)
class Work:
    request_id: int
    start: int
    tokens: tuple


class Scheduler:
    def __init__(self, cache, *, token_budget=128, prefill_chunk=64, max_active=4):
        if any(type(n) is not int or n < 1 for n in (token_budget, prefill_chunk, max_active)):
            raise ValueError('scheduler budgets must be positive integers')
        self.cache, self.token_budget, self.prefill_chunk, self.max_active = cache, token_budget, prefill_chunk, max_active
        self.requests, self.waiting, self.active = {}, deque(), deque()

    def add(self, request):
        if request.id in self.requests:
            raise ValueError('duplicate request ID')
        if not self.cache.fits_at_all(request.cache_limit):
            raise ValueError('request exceeds total KV capacity; reduce tokens or increase pages')
        self.requests[request.id] = request
        self.waiting.append(request.id)

    def plan(self):
        for _ in range(len(self.waiting)):
            if len(self.active) >= self.max_active:
                break
            request_id = self.waiting.popleft()
            request = self.requests[request_id]
            if self.cache.admit(request_id, request.cache_limit):
                request.state = 'active'
                self.active.append(request_id)
            else:
                self.waiting.append(request_id)
        remaining, work = self.token_budget, []
        for _ in range(len(self.active)):
            if not remaining:
                break
            request_id = self.active.popleft()
            request = self.requests[request_id]
            at, prompt_length = request.computed, len(request.prompt)
            chunk = self.prefill_chunk if at < prompt_length else 1
            count = min(chunk, remaining, prompt_length + len(request.output) - at)
            if count <= 0:
                raise RuntimeError('active request has no input to compute')
            if at + count <= prompt_length:           # slices, not prompt + output: that copy grows with the context
                tokens = request.prompt[at:at + count]
            elif at >= prompt_length:
                tokens = request.output[at - prompt_length:at - prompt_length + count]
            else:
                tokens = request.prompt[at:] + request.output[:at + count - prompt_length]
            work.append(Work(request_id, at, tuple(tokens)))
            remaining -= count
            self.active.append(request_id)
        if not work and self.waiting:
            raise RuntimeError('no runnable request despite an empty active set')
        return work

    def retire(self, request_id, state, reason):
        request = self.requests[request_id]
        if request.state not in ('waiting', 'active'):
            return False
        if request_id in self.waiting:
            self.waiting.remove(request_id)
        if request_id in self.active:
            self.active.remove(request_id)
            self.cache.release(request_id)
        request.state, request.finish_reason = state, reason
        return True

    @property
    def idle(self):
        return not self.waiting and not self.active
