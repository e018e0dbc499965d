"""The scheduler's decisions on the CPU, driven by a fake step function that keeps a simulated
cache: every page slot remembers the token written to it, and the "model" computes the next
token from what it reads back through the block tables. A wrong page, a stale page or a lost
token changes the output."""
import random
import zlib

import pytest

from minivllm_amd.cache import CacheManager, GroupSpec
from minivllm_amd.parts import KeepAll, KeepWindow
from minivllm_amd.config import SamplingParams
from minivllm_amd.engine.request import Request, RequestState
from minivllm_amd.engine.scheduler import Scheduler

VOCAB = 97
EOS = 5


def next_token(context):
    """The fake model: a function of the whole context."""
    return zlib.crc32(bytes(str(list(context)), "ascii")) % VOCAB


def expected_output(prompt, max_tokens, ignore_eos=True):
    toks, out = list(prompt), []
    while len(out) < max_tokens:
        t = next_token(toks)
        toks.append(t); out.append(t)
        if t == EOS and not ignore_eos:
            break
    return out


class FakeEngine:
    def __init__(self, num_pages, page_size, groups=None, max_tokens=64, max_seqs=8, chunk=None, prefix=False,
                 max_model_len=4096, repeat=1):
        self.groups = groups or [GroupSpec(KeepAll(), (0,))]
        self.manager = CacheManager(self.groups, num_pages, page_size, max_seqs, enable_prefix_caching=prefix)
        self.sched = Scheduler(self.manager, max_tokens, max_seqs, max_model_len, eos_token_ids=(EOS,),
                               prefill_chunk=chunk, max_decode_repeat=repeat)
        self.ps = page_size
        self.mem = [dict() for _ in self.groups]          # per group: (page, slot) -> token
        self.steps = []

    def run_step(self):
        step = self.sched.schedule()
        if step is None:
            return None
        return self.run_scheduled(step)

    def run_scheduled(self, step):
        assert step.num_tokens <= self.sched.max_num_batched_tokens
        assert len(step.seqs) <= self.sched.max_num_batched_seqs
        assert len({s.request.id for s in step.seqs}) == len(step.seqs)
        sampled = []
        if step.repeat > 1:
            sampled = self.device_runs(step)
            self.steps.append(step)
            done = self.sched.update(step, sampled)
            self.manager.check_invariants()
            return step, done
        for s in step.seqs:
            r = s.request
            seq = self.manager.sequence(r.id)
            assert s.start == seq.num_computed
            assert 1 <= s.num_tokens <= len(r.tokens) - s.start
            for g, spec in enumerate(self.groups):
                table = seq.pages[g]
                for pos in range(s.start, s.start + s.num_tokens):
                    page = table[pos // self.ps]
                    assert page >= 0
                    self.mem[g][(page, pos % self.ps)] = r.tokens[pos]
            if s.sample:
                end = s.start + s.num_tokens
                assert end == len(r.tokens)
                contexts = []
                for g, spec in enumerate(self.groups):
                    lo = spec.retention.first_kept_page(end - 1, 1)          # (page size 1: the first kept position)
                    table = seq.pages[g]
                    ctx = [self.mem[g][(table[p // self.ps], p % self.ps)] for p in range(lo, end)]
                    assert ctx == r.tokens[lo:end], "the cache does not hold the request's tokens"
                    contexts.append(ctx)
                sampled.append(next_token(contexts[0]))
            else:
                sampled.append(None)
        self.steps.append(step)
        done = self.sched.update(step, sampled)
        self.manager.check_invariants()
        return step, done

    def device_runs(self, step, before=None):
        """The device's part of a step that runs several times in a row: every run writes the
        newest token and draws the next from the cache. ``before``: what the launch before drew for
        the same requests, which the host has not recorded yet (a step scheduled ahead)."""
        assert not self.sched.waiting and all(s.is_decode and s.sample for s in step.seqs)
        sampled = []
        for i, s in enumerate(step.seqs):
            r = s.request
            seq = self.manager.sequence(r.id)
            toks, drawn = list(r.tokens) + (before[i] if before else []), []
            assert s.start == len(toks) - 1 and seq.num_computed == len(r.tokens) - 1
            assert r.num_completion_tokens + len(toks) - len(r.tokens) + step.repeat <= r.sampling_params.max_tokens
            for j in range(step.repeat):
                pos = s.start + j
                contexts = []
                for g, spec in enumerate(self.groups):
                    table = seq.pages[g]
                    assert table[pos // self.ps] >= 0
                    self.mem[g][(table[pos // self.ps], pos % self.ps)] = toks[pos]
                    lo = spec.retention.first_kept_page(pos, 1)
                    ctx = [self.mem[g][(table[p // self.ps], p % self.ps)] for p in range(lo, pos + 1)]
                    assert ctx == toks[lo:pos + 1], "the cache does not hold the request's tokens"
                    contexts.append(ctx)
                t = next_token(contexts[0])
                toks.append(t); drawn.append(t)
            sampled.append(drawn)
        return sampled

    def run_all_launching_ahead(self, limit=100000, each_round=None):
        """As an engine that launches the next step of decoded tokens before it has read the
        tokens of the one that runs. Returns how many steps were scheduled ahead.
        ``each_round(n)`` is called before round n (to submit requests meanwhile)."""
        ahead_count = n = 0
        in_flight = None                                   # (step, what the device drew)
        while in_flight is not None or not self.sched.finished:
            n += 1
            assert n < limit, "the scheduler does not terminate"
            if each_round is not None:
                each_round(n)
            if in_flight is None:
                step = self.sched.schedule()
                assert step is not None
                if step.repeat == 1:
                    self.run_scheduled(step)
                    continue
                in_flight = (step, self.device_runs(step))
            step, drawn = in_flight
            in_flight = None
            nxt = self.sched.schedule_ahead(step)
            if nxt is not None:
                ahead_count += 1
                assert nxt.repeat == step.repeat and [s.request for s in nxt.seqs] == [s.request for s in step.seqs]
                in_flight = (nxt, self.device_runs(nxt, before=drawn))
            self.steps.append(step)
            self.sched.update(step, drawn)
            self.manager.check_invariants()
        return ahead_count

    def run_all(self, limit=100000):
        n = 0
        while not self.sched.finished:
            assert self.run_step() is not None
            n += 1
            assert n < limit, "the scheduler does not terminate"
        return n


def submit(engine, prompt, **sp):
    r = Request(prompt, SamplingParams(temperature=0.0, **sp))
    engine.sched.submit(r)
    return r


def test_mixed_steps_and_token_budget():
    e = FakeEngine(num_pages=64, page_size=4, max_tokens=16, max_seqs=8)
    rng = random.Random(1)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=6, ignore_eos=True)
            for n in (5, 17, 33, 1)]
    e.run_all()
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, 6)
        assert r.finish_reason == "length" and r.state == RequestState.FINISHED
    # the 33-token prompt was cut into portions under the budget of 16, beside other work
    long_portions = [s.num_tokens for st in e.steps for s in st.seqs if s.request is reqs[2] and not s.is_decode]
    assert len(long_portions) >= 3 and sum(long_portions) == 33 and max(long_portions) <= 16
    assert any(any(s.is_decode for s in st.seqs) and any(not s.is_decode for s in st.seqs) for st in e.steps), \
        "no step mixed decoded tokens with a prompt portion"
    assert all(p.num_free == p.num_pages for p in e.manager.pools)


def test_prefill_chunk_and_first_come_first_served():
    e = FakeEngine(num_pages=64, page_size=8, max_tokens=64, max_seqs=2, chunk=7)
    rng = random.Random(2)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=3, ignore_eos=True) for n in (20, 9, 4)]
    e.run_all()
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, 3)
    assert max(s.num_tokens for st in e.steps for s in st.seqs) <= 7
    first_step_of = {r.id: next(i for i, st in enumerate(e.steps) if r in st.requests) for r in reqs}
    assert first_step_of[reqs[0].id] <= first_step_of[reqs[1].id] <= first_step_of[reqs[2].id]
    # only two requests may run at once: the third waits until one finishes
    assert all(len(st.seqs) <= 2 for st in e.steps)


def test_eos_stops_unless_ignored():
    # find a prompt whose greedy continuation hits EOS early
    rng = random.Random(3)
    while True:
        prompt = [rng.randrange(VOCAB) for _ in range(6)]
        out = expected_output(prompt, 40, ignore_eos=False)
        if len(out) < 40:
            break
    e = FakeEngine(num_pages=64, page_size=4)
    a = submit(e, prompt, max_tokens=40)
    b = submit(e, prompt, max_tokens=40, ignore_eos=True)
    e.run_all()
    assert a.completion_tokens == out and a.completion_tokens[-1] == EOS and a.finish_reason == "stop"
    assert len(b.completion_tokens) == 40 and b.finish_reason == "length"


@pytest.mark.parametrize("seed", range(4))
def test_preemption_under_page_pressure(seed):
    """So few pages that running requests must give way; every request still gets exactly its
    tokens, identical to running it alone (minivllm/scheduler/scheduler.py:66-72,91-98)."""
    rng = random.Random(seed)
    ps = 4
    e = FakeEngine(num_pages=14, page_size=ps, max_tokens=32, max_seqs=6)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(rng.randint(1, 20))], max_tokens=rng.randint(4, 24),
                   ignore_eos=True) for _ in range(7)]
    e.run_all()
    assert e.sched.num_preemptions > 0, "the test did not create page pressure"
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, r.sampling_params.max_tokens)
    assert all(p.num_free == p.num_pages for p in e.manager.pools) and e.manager.slots.num_free == 6


def test_preempted_request_returns_to_the_front_and_the_newest_gives_way():
    ps = 4
    e = FakeEngine(num_pages=6, page_size=ps, max_tokens=64, max_seqs=4)
    a = submit(e, [1] * 7, max_tokens=12, ignore_eos=True)      # may reach 19 tokens = 5 pages
    b = submit(e, [2] * 7, max_tokens=12, ignore_eos=True)      # together they would need 10 of 6
    e.run_step()
    assert [r.id for r in e.sched.running] == [a.id, b.id]
    c = submit(e, [3] * 3, max_tokens=2, ignore_eos=True)       # arrives later, waits behind a preempted b
    while b.num_preemptions == 0:
        e.run_step()
    assert a.num_preemptions == 0                  # the newer one gave way
    assert b.state in (RequestState.WAITING, RequestState.RUNNING)
    if b.state == RequestState.WAITING:
        assert e.sched.waiting[0] is b and b.id not in e.manager   # back at the front, before c
    e.run_all()
    for r in (a, b, c):
        assert r.completion_tokens == expected_output(r.prompt_tokens, r.sampling_params.max_tokens)
    assert b.finish_time >= a.finish_time or b.num_preemptions > 0


def test_windowed_group_and_recycled_pages():
    groups = [GroupSpec(KeepAll(), (0,)), GroupSpec(KeepWindow(6), (1,))]
    e = FakeEngine(num_pages=40, page_size=4, groups=groups, max_tokens=24, max_seqs=4)
    rng = random.Random(5)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=20, ignore_eos=True) for n in (30, 3, 18, 9, 25)]
    e.run_all()
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, 20)


def test_prefix_reuse_skips_cached_pages():
    e = FakeEngine(num_pages=64, page_size=4, prefix=True, max_tokens=64)
    shared = list(range(10, 26))                   # 16 tokens = 4 full pages
    a = submit(e, shared + [1, 2, 3], max_tokens=4, ignore_eos=True)
    e.run_all()
    b = submit(e, shared + [7, 8], max_tokens=4, ignore_eos=True)
    e.run_step()
    first = next(s for s in e.steps[-1].seqs if s.request is b)
    assert first.start == 16 and first.num_tokens == 2          # the shared pages were not run again
    e.run_all()
    assert a.completion_tokens == expected_output(a.prompt_tokens, 4)
    assert b.completion_tokens == expected_output(b.prompt_tokens, 4)
    # a prompt that is cached entirely still computes its last token
    c = submit(e, shared, max_tokens=2, ignore_eos=True)
    e.run_step()
    first = next(s for s in e.steps[-1].seqs if s.request is c)
    assert first.start == 12 and first.num_tokens == 4
    e.run_all()
    assert c.completion_tokens == expected_output(shared, 2)


def test_refused_at_submit():
    e = FakeEngine(num_pages=4, page_size=4, max_model_len=64)
    with pytest.raises(ValueError, match="max_model_len"):
        submit(e, [1] * 64, max_tokens=1)
    with pytest.raises(ValueError, match="pages"):
        submit(e, [1] * 10, max_tokens=30)          # 40 tokens = 10 pages, the pool has 4
    with pytest.raises(ValueError):
        Request([], SamplingParams())


def test_max_model_len_ends_a_request():
    e = FakeEngine(num_pages=64, page_size=4, max_model_len=12)
    r = submit(e, [1, 2, 3, 4, 5], max_tokens=100, ignore_eos=True)
    e.run_all()
    assert len(r.tokens) == 12 and r.finish_reason == "length"


def test_decode_steps_run_in_a_row():
    """Steps of decoded tokens only may run several times before the host looks: same tokens as one
    by one, never past max_tokens, tokens drawn after an end token are dropped, and a waiting
    request is admitted at the next step."""
    rng = random.Random(11)
    prompts = [[rng.randrange(VOCAB) for _ in range(n)] for n in (5, 17, 9, 2, 30)]
    limits = [13, 7, 40, 1, 22]
    for use_eos in (False, True):
        e = FakeEngine(num_pages=64, page_size=4, max_tokens=32, max_seqs=4, repeat=4)
        reqs = [submit(e, p, max_tokens=m, ignore_eos=not use_eos) for p, m in zip(prompts[:3], limits[:3])]
        late = []
        n = 0
        while not e.sched.finished:
            step, _ = e.run_step()
            n += 1
            if n == 6:                                   # arrive while the others decode
                late = [submit(e, p, max_tokens=m, ignore_eos=not use_eos) for p, m in zip(prompts[3:], limits[3:])]
                assert e.sched.schedule is not None
            assert n < 1000
        for r, m in zip(reqs + late, limits):
            assert r.completion_tokens == expected_output(r.prompt_tokens, m, ignore_eos=not use_eos)
        repeats = [st.repeat for st in e.steps]
        assert max(repeats) == 4 and 1 in repeats
        # the step after the late arrival took them in: nobody waits while steps repeat
        assert all(st.repeat == 1 or all(s.is_decode for s in st.seqs) for st in e.steps)
        assert all(p.num_free == p.num_pages for p in e.manager.pools)


def test_decode_steps_list_the_longest_contexts_first():
    """A step of decoded tokens only names its requests by falling context length (the attention's
    workgroups start in that order); steps with prompt portions keep the order of arrival; the tokens
    are what they are in any order."""
    rng = random.Random(5)
    lengths = (7, 30, 3, 18, 30, 11)
    e = FakeEngine(num_pages=128, page_size=4, max_tokens=64, max_seqs=8, repeat=2)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=9 + i, ignore_eos=True) for i, n in enumerate(lengths)]
    n = 0
    while not e.sched.finished:
        e.run_step()
        n += 1
        assert n < 1000
    decode_steps = [st for st in e.steps if all(s.is_decode for s in st.seqs)]
    assert decode_steps and any(len(st.seqs) == len(lengths) for st in decode_steps)
    for st in decode_steps:
        starts = [s.start for s in st.seqs]
        assert starts == sorted(starts, reverse=True)
    first = e.steps[0]
    assert [s.request.id for s in first.seqs] == [r.id for r in reqs][:len(first.seqs)]
    for i, r in enumerate(reqs):
        assert r.completion_tokens == expected_output(r.prompt_tokens, 9 + i, ignore_eos=True)


def test_no_row_of_steps_without_the_pages_for_all_of_it():
    """With pages for fewer positions than a full row needs, the step runs once (a row has the full
    length or none: the executor keeps two graphs per size, not one per length); nothing is
    preempted for the sake of repeating."""
    e = FakeEngine(num_pages=5, page_size=4, max_tokens=32, max_seqs=4, repeat=8)
    rng = random.Random(12)
    a = submit(e, [rng.randrange(VOCAB) for _ in range(7)], max_tokens=12, ignore_eos=True)
    b = submit(e, [rng.randrange(VOCAB) for _ in range(6)], max_tokens=3, ignore_eos=True)
    e.run_all()
    assert a.completion_tokens == expected_output(a.prompt_tokens, 12)
    assert b.completion_tokens == expected_output(b.prompt_tokens, 3)
    assert e.sched.num_preemptions == 0
    assert all(st.repeat in (1, 8) for st in e.steps) and any(st.repeat == 1 and all(s.is_decode for s in st.seqs)
                                                              for st in e.steps)
    assert all(p.num_free == p.num_pages for p in e.manager.pools)


def test_repeat_with_a_window_group():
    groups = [GroupSpec(KeepAll(), (0,)), GroupSpec(KeepWindow(6), (1,))]
    e = FakeEngine(num_pages=48, page_size=4, groups=groups, max_tokens=32, max_seqs=4, repeat=4)
    rng = random.Random(13)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=19, ignore_eos=True) for n in (11, 3)]
    e.run_all()
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, 19)
    assert max(st.repeat for st in e.steps) == 4
    assert all(p.num_free == p.num_pages for p in e.manager.pools)


@pytest.mark.parametrize("use_eos", [False, True])
@pytest.mark.parametrize("seed", range(6))
def test_steps_scheduled_ahead_give_the_same_tokens(seed, use_eos):
    """The next step of decoded tokens is launched before the tokens of the running one are known:
    the same tokens as step by step; what ran on for a request that ended on an end token is
    dropped with its pages; near max_tokens, max_model_len or the pool's end nothing is launched
    ahead."""
    rng = random.Random(100 + seed)
    prompts = [[rng.randrange(VOCAB) for _ in range(rng.randrange(1, 30))] for _ in range(7)]
    limits = [rng.randrange(1, 60) for _ in prompts]
    e = FakeEngine(num_pages=rng.choice([40, 64, 200]), page_size=4, max_tokens=32, max_seqs=rng.choice([2, 4, 8]),
                   repeat=rng.choice([2, 4]), max_model_len=rng.choice([50, 4096]))
    reqs = [submit(e, p, max_tokens=m, ignore_eos=not use_eos) for p, m in zip(prompts, limits)]
    ahead = e.run_all_launching_ahead()
    for r, m in zip(reqs, limits):
        want = expected_output(r.prompt_tokens, min(m, 50 - len(r.prompt_tokens)) if e.sched.max_model_len == 50 else m,
                               ignore_eos=not use_eos)
        assert r.completion_tokens == want, (r.id, ahead)
        assert r.state == RequestState.FINISHED
    assert all(p.num_free == p.num_pages for p in e.manager.pools)
    assert e.manager.slots.num_free == e.manager.slots.num_slots if hasattr(e.manager.slots, "num_slots") else True


def test_steps_are_scheduled_ahead_when_nothing_can_change():
    e = FakeEngine(num_pages=64, page_size=4, max_tokens=32, max_seqs=4, repeat=4)
    rng = random.Random(5)
    reqs = [submit(e, [rng.randrange(VOCAB) for _ in range(n)], max_tokens=41, ignore_eos=True) for n in (3, 9)]
    ahead = e.run_all_launching_ahead()
    assert ahead >= 7                        # 41 tokens = 1 + 10 steps of 4, all but the last launched ahead
    for r in reqs:
        assert r.completion_tokens == expected_output(r.prompt_tokens, 41)
    # fewer tokens to go than both steps draw, or fewer free pages than both need: nothing is
    # launched ahead and nothing is reserved
    for pages, limit in ((64, 7), (5, 9)):
        e = FakeEngine(num_pages=pages, page_size=4, max_tokens=32, max_seqs=2, repeat=4)
        a = submit(e, [1, 2, 3], max_tokens=limit, ignore_eos=True)
        b = submit(e, [4, 5, 6], max_tokens=limit, ignore_eos=True)
        e.run_scheduled(e.sched.schedule())      # the prompts
        step = e.sched.schedule()
        assert step.repeat == 4 and not e.sched.waiting
        free = [p.num_free for p in e.manager.pools]
        assert e.sched.schedule_ahead(step) is None and [p.num_free for p in e.manager.pools] == free
        e.sched.update(step, e.device_runs(step))
        e.run_all()
        assert a.completion_tokens == expected_output(a.prompt_tokens, limit)
        assert b.completion_tokens == expected_output(b.prompt_tokens, limit)


@pytest.mark.parametrize("seed", range(4))
def test_requests_that_arrive_while_a_step_is_in_flight(seed):
    """New requests come in while a step launched ahead is running: it is read first, then they are
    admitted; every request still gets the tokens of a run step by step."""
    rng = random.Random(200 + seed)
    e = FakeEngine(num_pages=120, page_size=4, max_tokens=24, max_seqs=6, repeat=4)
    first = [submit(e, [rng.randrange(VOCAB) for _ in range(rng.randrange(2, 20))], max_tokens=rng.randrange(20, 50),
                    ignore_eos=seed % 2 == 0) for _ in range(2)]
    late = []
    arrivals = {4: 1, 5: 2, 9: 1}

    def each_round(n):
        for _ in range(arrivals.get(n, 0)):
            late.append(submit(e, [rng.randrange(VOCAB) for _ in range(rng.randrange(1, 25))],
                               max_tokens=rng.randrange(1, 40), ignore_eos=seed % 2 == 0))

    ahead = e.run_all_launching_ahead(each_round=each_round)
    assert ahead > 0 and len(late) == 4
    for r in first + late:
        assert r.completion_tokens == expected_output(r.prompt_tokens, r.sampling_params.max_tokens,
                                                      ignore_eos=seed % 2 == 0)
    assert all(p.num_free == p.num_pages for p in e.manager.pools)
