"""The serving loop: plan -> one batched step -> sample -> events -> release.

Interface of the reference's ``Engine`` (qil/engine.py:12-154): ``submit``,
``step``, ``cancel``, ``result``, ``idle``, ``generate``, ``close``, with the same
arguments and result fields; ``submit``/``generate`` also take ``temperature`` and
``seed``.  The reference's ablation switches (batch_decode, selective_logits,
decode_attention) do not exist: there is one path.
"""
from time import perf_counter

from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .scheduler import Request, Scheduler
from .step import ModelRunner


class Engine:
    def __init__(self, model, *, num_pages=256, page_size=16, token_budget=128, prefill_chunk=64, max_active=4,
                 clock=perf_counter, runner=None, sampler=None):
        self.model, self.clock, self.next_id = model, clock, 0
        self.runner = runner or ModelRunner(model, num_pages=num_pages, page_size=page_size,
                                            max_requests=max_active, max_step_tokens=token_budget)
        self.cache = self.runner.cache
        self.sampler = sampler or Sampler()
        self.scheduler = Scheduler(self.cache, token_budget=token_budget, prefill_chunk=prefill_chunk,
                                   max_active=max_active)
        self.steps = 0

    def submit(self, prompt, *, max_new_tokens=64, ignore_eos=False, temperature=0.0, seed=0):
        prompt = list(prompt)
        vocab = self.model.vocab
        if not prompt or any(type(t) is not int or not 0 <= t < vocab for t in prompt):     # qil/engine.py:36-37
            raise ValueError('prompt must contain valid integer token IDs')
        if type(max_new_tokens) is not int or max_new_tokens < 1:
            raise ValueError('max_new_tokens must be a positive integer')
        limit = getattr(self.model.config, 'max_position_embeddings', None)
        if limit is not None and len(prompt) + max_new_tokens > limit:                       # qil/engine.py:40-41
            raise ValueError('request exceeds model context length')
        params = SamplingParams(temperature, seed)
        eos = frozenset() if ignore_eos else frozenset(getattr(self.model.config, 'eos_ids', ()))
        request_id = self.next_id
        self.scheduler.add(Request(request_id, prompt, max_new_tokens, eos, self.clock(),
                                   temperature=params.temperature, seed=params.seed))
        self.next_id += 1
        return request_id

    def step(self):
        """Execute one budgeted plan as one batch; events of the tokens it produced."""
        plan = self.scheduler.plan()
        if not plan:
            return []
        requests = self.scheduler.requests
        ready = [w.start + len(w.tokens) == len(requests[w.request_id].prompt) + len(requests[w.request_id].output)
                 for w in plan]
        try:
            entries = [StepEntry(w.request_id, w.tokens, (len(w.tokens) - 1,) if r else ())
                       for w, r in zip(plan, ready)]
            rows = [requests[w.request_id] for w, r in zip(plan, ready) if r]
            params, counters = [SamplingParams(q.temperature, q.seed) for q in rows], [len(q.output) for q in rows]
            fused = getattr(self.runner, 'step_and_sample', None)
            if fused is not None and isinstance(self.sampler, Sampler):     # the draw rides in the step's launches
                emitted = iter(fused(entries, self.sampler, params, counters))
            else:
                logits = self.runner.step(entries)
                emitted = iter(self.sampler.sample(logits, params, counters) if logits is not None else ())
        except Exception as error:
            # The failed batch may have written part of its keys and values: retire every member
            # so that none resumes from a partial cache (qil/engine.py:87-93).
            for work in plan:
                requests[work.request_id].error = str(error)
                self.scheduler.retire(work.request_id, 'failed', 'error')
            raise
        self.steps += 1
        events = []
        for work, is_ready in zip(plan, ready):
            event = self._complete_work(work, next(emitted) if is_ready else None)
            if event is not None:
                events.append(event)
        return events

    def _complete_work(self, work, token):
        request = self.scheduler.requests[work.request_id]
        request.computed = work.start + len(work.tokens)
        if token is None:
            return None
        observed = self.clock()
        request.output.append(token)
        request.token_times_s.append(observed)
        reason = 'eos' if token in request.eos else (
            'length' if len(request.output) == request.max_new_tokens else None)
        if reason:
            self.scheduler.retire(request.id, 'completed', reason)
        return dict(request_id=request.id, token_id=token, timestamp_s=observed, finished=reason is not None)

    def cancel(self, request_id):
        return self.scheduler.retire(request_id, 'cancelled', 'cancelled')

    def result(self, request_id):
        request = self.scheduler.requests[request_id]
        times = request.token_times_s
        gaps = [b - a for a, b in zip(times, times[1:])]
        return dict(
            request_id=request_id, state=request.state, finish_reason=request.finish_reason,
            error=request.error, token_ids=list(request.output),
            token_times_s=[t - request.arrival_s for t in times],
            ttft_s=times[0] - request.arrival_s if times else None,
            e2e_s=times[-1] - request.arrival_s if request.state == 'completed' else None,
            tpot_s=sum(gaps) / len(gaps) if gaps else None)

    @property
    def idle(self):
        return self.scheduler.idle

    def generate(self, prompts, *, max_new_tokens=64, ignore_eos=False, temperature=0.0, seed=0):
        if not self.idle:
            raise ValueError('generate requires an idle engine; use submit/step for live requests')
        request_ids = []
        try:
            for index, prompt in enumerate(prompts):
                request_ids.append(self.submit(prompt, max_new_tokens=max_new_tokens, ignore_eos=ignore_eos,
                                               temperature=temperature, seed=seed + index))
            while not self.idle:
                self.step()
        except Exception:
            for request_id in request_ids:
                self.cancel(request_id)
            raise
        return [self.result(request_id) for request_id in request_ids]

    def close(self):
        for request_id in list(self.scheduler.active) + list(self.scheduler.waiting):
            self.cancel(request_id)
