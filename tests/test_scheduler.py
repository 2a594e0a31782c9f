"""The scheduler's decisions, and the serving loop around a fake step function (CPU)."""
import pytest
import torch

from qil_amd.cache import CacheManager
from qil_amd.engine import Engine, Request, Scheduler
from qil_amd.parts import KVNeed


class FakeModel:
    """Enough of a model for the serving loop: a vocabulary, a config, and logits that make the next
    token a known function of the last one."""
    vocab = 50

    class config:
        max_position_embeddings = 64
        eos_ids = frozenset({49})


class FakeRunner:
    def __init__(self, pages=16, page_size=4, requests=4, fail_on=None):
        self.cache = CacheManager([KVNeed(1, 8, None)], num_pages=pages, page_size=page_size, max_requests=requests,
                                  allocate=False)
        self.batches, self.fail_on = [], fail_on

    def step(self, entries):
        self.batches.append([(e.request, len(e.tokens), e.want) for e in entries])
        for e in entries:
            start = self.cache.computed[e.request]
            self.cache.ensure(e.request, start + len(e.tokens))
            self.cache.advance(e.request, start + len(e.tokens))
        if self.fail_on is not None and len(self.batches) == self.fail_on:
            raise RuntimeError('injected failure after the cache was written')
        rows = [e.tokens[w] for e in entries for w in e.want]
        if not rows:
            return None
        logits = torch.zeros(len(rows), FakeModel.vocab)
        for i, token in enumerate(rows):
            logits[i, (token * 7 + 3) % 48] = 5.0          # next token; never the eos id 49
        return logits


class FakeSampler:
    def sample(self, logits, params, counters):
        return logits.argmax(-1).tolist()


def engine(**kwargs):
    runner = kwargs.pop('runner', None) or FakeRunner()
    return Engine(FakeModel(), runner=runner, sampler=FakeSampler(), **kwargs), runner


def follow(token, count):
    out = []
    for _ in range(count):
        token = (token * 7 + 3) % 48
        out.append(token)
    return out


def test_budget_chunks_and_round_robin():
    """qil/scheduler.py:68-84: one piece of work per active request, cut to the budget, served ones go last."""
    e, runner = engine(token_budget=7, prefill_chunk=4, max_active=3)
    ids = [e.submit([1] * 9, max_new_tokens=2, ignore_eos=True), e.submit([2] * 2, max_new_tokens=2, ignore_eos=True),
           e.submit([3] * 6, max_new_tokens=2, ignore_eos=True)]
    e.step()
    assert runner.batches[0] == [(0, 4, ()), (1, 2, (1,)), (2, 1, ())]             # 4 + 2 + 1 = budget 7; prompt 1 is complete
    e.step()
    assert runner.batches[1] == [(0, 4, ()), (1, 1, (0,)), (2, 2, ())]             # 1 decodes its one token; 2 cut to the rest
    assert all(sum(n for _, n, _ in batch) <= 7 for batch in runner.batches)
    while not e.idle:
        e.step()
    for rid, first in zip(ids, (1, 2, 3)):
        result = e.result(rid)
        assert result['token_ids'] == follow(first, 2) and result['finish_reason'] == 'length'
    assert runner.cache.free_pages == [16] and not runner.cache.slots


def test_no_starvation_with_a_budget_of_one():
    """tests/qil/test_engine.py:66-73."""
    e, _ = engine(token_budget=1, prefill_chunk=1)
    ids = [e.submit([1], max_new_tokens=3, ignore_eos=True) for _ in range(3)]
    events = []
    while not e.idle:
        events.extend(e.step())
    assert [event['request_id'] for event in events] == ids * 3


@pytest.mark.parametrize('budget,chunk,pages', [(1, 1, 16), (5, 3, 16), (8, 8, 4)])   # tests/qil/test_engine.py:17
def test_outputs_do_not_depend_on_budget_chunk_or_pages(budget, chunk, pages):
    e, runner = engine(runner=FakeRunner(pages=pages), token_budget=budget, prefill_chunk=chunk, max_active=3)
    prompts = [[1, 2, 3, 4, 5], [8], [5, 3, 2]]
    results = e.generate(prompts, max_new_tokens=5, ignore_eos=True)
    assert [r['token_ids'] for r in results] == [follow(p[-1], 5) for p in prompts]
    assert all(r['state'] == 'completed' and len(r['token_times_s']) == 5 for r in results)
    assert all(len(batch) <= 3 and sum(n for _, n, _ in batch) <= budget for batch in runner.batches)
    assert runner.cache.free_pages == [pages]


def test_when_pages_run_out_requests_wait_or_are_refused():
    """Admission reserves a request's whole life (qil/cache.py:54-68), so pages cannot run out inside
    one: lack of room shows as waiting, and a request that could never fit is refused at submit."""
    e, runner = engine(runner=FakeRunner(pages=4, page_size=4), token_budget=8, prefill_chunk=8, max_active=4)
    big = e.submit([1] * 10, max_new_tokens=3, ignore_eos=True)                  # 12 cached tokens: 3 pages
    small = e.submit([2] * 5, max_new_tokens=4, ignore_eos=True)                 # 8 tokens: 2 pages -> must wait
    tiny = e.submit([3], max_new_tokens=2, ignore_eos=True)                      # 2 tokens: 1 page -> overtakes
    e.step()
    assert e.result(big)['state'] == 'active' and e.result(small)['state'] == 'waiting'
    assert e.result(tiny)['state'] == 'active'
    with pytest.raises(ValueError, match='capacity'):
        e.submit([1] * 16, max_new_tokens=2)                                     # 17 tokens: 5 pages > 4
    while not e.idle:
        e.step()
        runner.cache.check()
    assert all(e.result(r)['state'] == 'completed' for r in (big, small, tiny))
    assert runner.cache.free_pages == [4]


def test_eos_cancel_and_dynamic_arrival():
    e, runner = engine(token_budget=4, prefill_chunk=4)
    first = e.submit([1, 2, 3], max_new_tokens=5)
    e.step()
    second = e.submit([8], max_new_tokens=2)
    assert e.cancel(first) and not e.cancel(first)                              # idempotent (qil/engine.py:117-118)
    while not e.idle:
        e.step()
    assert e.result(first)['state'] == 'cancelled' and e.result(second)['token_ids'] == follow(8, 2)
    FakeModel.config.eos_ids = frozenset({follow(8, 1)[0]})
    try:
        result = e.generate([[8]], max_new_tokens=5)[0]
        assert result['finish_reason'] == 'eos' and len(result['token_ids']) == 1 and result['tpot_s'] is None
        assert len(e.generate([[8]], max_new_tokens=3, ignore_eos=True)[0]['token_ids']) == 3
    finally:
        FakeModel.config.eos_ids = frozenset({49})
    assert not runner.cache.slots


def test_failure_retires_the_batch_and_the_rest_goes_on():
    """qil/engine.py:87-93 and tests/qil/test_engine.py:47-63."""
    runner = FakeRunner(fail_on=2)
    e, _ = engine(runner=runner, max_active=1, token_budget=4, prefill_chunk=4)
    active = e.submit([1, 2], max_new_tokens=3, ignore_eos=True)
    waiting = e.submit([3], max_new_tokens=3, ignore_eos=True)
    e.step()
    assert e.result(waiting)['state'] == 'waiting'
    with pytest.raises(RuntimeError, match='injected'):
        e.step()
    failed = e.result(active)
    assert failed['state'] == 'failed' and 'injected' in failed['error'] and failed['e2e_s'] is None
    assert not runner.cache.slots and runner.cache.free_pages == [16]            # every page is back
    while not e.idle:
        e.step()
    assert e.result(waiting)['token_ids'] == follow(3, 3)


@pytest.mark.parametrize('prompt,count', [([], 1), ([-1], 1), ([50], 1), ([True], 1), ([1], 0), ([1], 64)])
def test_bad_requests_are_refused_before_anything_is_taken(prompt, count):     # tests/qil/test_engine.py:76-81
    e, runner = engine()
    with pytest.raises(ValueError):
        e.submit(prompt, max_new_tokens=count)
    assert e.idle and not runner.cache.slots
    for bad in (dict(temperature=-1.0), dict(temperature=float('nan')), dict(seed=1.5)):
        with pytest.raises(ValueError):
            e.submit([1], **bad)


def test_generate_cleans_up_after_a_refusal():
    e, runner = engine(runner=FakeRunner(pages=2, page_size=4))
    with pytest.raises(ValueError, match='capacity'):
        e.generate([[1], [1] * 8], max_new_tokens=2)
    assert e.idle and not runner.cache.slots
    e.submit([1], max_new_tokens=2)
    with pytest.raises(ValueError, match='idle'):
        e.generate([[2]], max_new_tokens=2)
    e.close()
    assert e.idle


def test_scheduler_rejects_nonsense():
    cache = CacheManager([KVNeed(1, 8, None)], num_pages=2, page_size=2, max_requests=2, allocate=False)
    for bad in (dict(token_budget=0), dict(prefill_chunk=-1), dict(max_active=1.5)):
        with pytest.raises(ValueError):
            Scheduler(cache, **bad)
    scheduler = Scheduler(cache)
    scheduler.add(Request(0, [1], 1, frozenset(), 0.0))
    with pytest.raises(ValueError, match='duplicate'):
        scheduler.add(Request(0, [1], 1, frozenset(), 0.0))


def test_counters_of_the_loop():
    e, runner = engine(token_budget=6, prefill_chunk=4, max_active=2)
    assert e.stats()['steps'] == 0 and e.stats()['pages_in_use'] == [0]
    e.submit([1] * 9, max_new_tokens=2, ignore_eos=True)
    e.submit([2] * 3, max_new_tokens=3, ignore_eos=True)
    e.submit([3], max_new_tokens=1, ignore_eos=True)
    e.step()
    stats = e.stats()
    assert stats['steps'] == 1 and stats['last_step_tokens'] == 6 and stats['last_step_requests'] == 2
    assert stats['active'] == 2 and stats['waiting'] == 1 and stats['drawn'] == 0
    assert stats['pages_in_use'] == [2] and stats['pages_total'] == [16]      # 4 + 2 tokens in pages of 4
    while not e.idle:
        e.step()
    stats = e.stats()
    assert stats['tokens'] == (9 + 1) + (3 + 2) + 1 and stats['drawn'] == 6   # fed: prompts and all drawn tokens but the last
    assert stats['pages_in_use'] == [0] and stats['peak_pages_in_use'] >= 4 and stats['active'] == stats['waiting'] == 0


def test_requests_report_phases():
    from qil_amd.engine import Phase
    e, _ = engine()
    rid = e.submit([1, 2], max_new_tokens=1, ignore_eos=True)
    request = e.scheduler.requests[rid]
    assert request.phase is Phase.WAITING and e.result(rid)['state'] == 'waiting' and e.result(rid)['ttft_s'] is None
    e.step()
    assert request.phase is Phase.COMPLETED and e.result(rid)['finish_reason'] == 'length'
    assert request.span(0, 3) == (1, 2, follow(2, 1)[0]) and request.span(2, 3) == (follow(2, 1)[0],)
