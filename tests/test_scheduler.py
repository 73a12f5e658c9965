"""The scheduler's decisions, with the real cache manager and a step function
that computes nothing (the next token is a function of the tokens fed)."""
import numpy as np
import pytest

from kipp_amd.cache import CacheManager, KVNeed
from kipp_amd.engine.scheduler import Request, RequestRefused, Scheduler
from kipp_amd.sampling import SampleParams

VOCAB = 50


class FakeEngine:
    """Keeps the cache bookkeeping of the real engine; 'logits' are one-hot at
    (sum of the request's tokens so far) % VOCAB."""

    def __init__(self, num_pages=8, page_size=4, max_requests=4, max_position=64, share=True):
        self.cache = CacheManager([KVNeed(1, 16)], [None], page_size, num_pages, max_requests, max_position,
                                  runtime=None, share_prefixes=share)
        self.vocab_size = VOCAB
        self.calls = []

    def step(self, entries, borrow=False):
        reqs = []
        for e in entries:
            if e.request not in self.cache.requests:
                self.cache.open(e.request)
            reqs.append(self.cache.requests[e.request])
        self.cache.reserve([(r, len(e.tokens)) for r, e in zip(reqs, entries)])
        rows = []
        for r, e in zip(reqs, entries):
            self.cache.commit(r, e.tokens)
            for w in e.want:
                row = np.zeros(VOCAB, dtype=np.float32)
                row[sum(r.tokens[:r.length - len(e.tokens) + w + 1]) % VOCAB] = 1.0
                rows.append(row)
        self.calls.append([(e.request, len(e.tokens), list(e.want)) for e in entries])
        self.cache.check()
        return np.stack(rows) if rows else None

    def choose(self, logits, requests):
        return [int(np.argmax(row)) for row in logits]

    def close(self, rid):
        self.cache.close(rid)


def expected_output(prompt, n, stop=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = sum(toks) % VOCAB
        if t in stop:
            break
        out.append(t)
        toks.append(t)
    return out


def test_one_request_prefill_in_portions_then_decode():
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng, max_step_tokens=8, prefill_chunk=5)
    prompt = list(range(1, 13))
    s.add(Request("a", prompt, 4))
    done = s.run()
    assert done["a"].output == expected_output(prompt, 4) and done["a"].finish_reason == "length"
    # portions of 5, 5, 2 (the last asks for its last place), then single tokens; the 4th token is never run
    assert eng.calls == [[("a", 5, [])], [("a", 5, [])], [("a", 2, [1])], [("a", 1, [0])], [("a", 1, [0])], [("a", 1, [0])]]
    assert eng.cache.free_pages() == [16] and s.stats.generated_tokens == 4 and s.stats.prompt_tokens == 12


def test_decode_tokens_come_first_and_the_budget_is_kept():
    eng = FakeEngine(num_pages=40, max_requests=4, share=False)
    s = Scheduler(eng, max_step_tokens=6, prefill_chunk=4)
    s.add(Request("a", [1, 2, 3], 6))
    s.step()                                              # a: whole prompt, first token
    s.add(Request("b", list(range(10)), 2))
    s.add(Request("c", list(range(5)), 2))
    s.step()
    assert eng.calls[-1] == [("a", 1, [0]), ("b", 4, []), ("c", 1, [])]   # 1 + 4 + 1 = budget 6
    for call in eng.calls:
        assert sum(n for _, n, _ in call) <= 6
    s.run()
    assert s.finished["b"].output == expected_output(list(range(10)), 2)
    assert s.finished["c"].output == expected_output(list(range(5)), 2)
    assert s.finished["a"].output == expected_output([1, 2, 3], 6)


def test_stop_token_is_neither_kept_nor_fed_back():
    prompt = [3, 4]
    chain = expected_output(prompt, 5)
    stop = chain[2]
    eng = FakeEngine()
    s = Scheduler(eng)
    s.add(Request("a", prompt, 10, stop_tokens=(stop,)))
    done = s.run()
    assert done["a"].output == chain[:2] and done["a"].finish_reason == "stop"
    assert sum(n for call in eng.calls for _, n, _ in call) == len(prompt) + 2   # the stop token was not run


def test_refusals():
    s = Scheduler(FakeEngine(num_pages=4, max_position=64))
    with pytest.raises(RequestRefused, match="positions"):
        s.add(Request("a", [1] * 60, 10))
    with pytest.raises(RequestRefused, match="pages"):
        s.add(Request("b", [1] * 20, 4))                  # 23 tokens need 6 pages, the pool has 4
    with pytest.raises(RequestRefused, match="vocabulary"):
        s.add(Request("c", [VOCAB], 1))
    with pytest.raises(RequestRefused, match="empty"):
        s.add(Request("d", [], 1))
    with pytest.raises(ValueError, match="top_p"):
        s.add(Request("e", [1], 1, SampleParams(temperature=1.0, top_p=0.0)))
    assert s.stats.refused == 3 and s.idle


def test_when_pages_run_out_requests_wait_in_order_and_nothing_is_corrupted():
    # 6 pages of 4 tokens.  a and b need 3 pages each at worst; c must wait although a slot is free.
    eng = FakeEngine(num_pages=6, max_requests=4, share=False)
    s = Scheduler(eng, max_step_tokens=64, prefill_chunk=64)
    pa, pb, pc, pd = [1] * 6, [2] * 7, [3] * 5, [4]
    s.add(Request("a", pa, 6))                            # budget 11 tokens -> 3 pages
    s.add(Request("b", pb, 5))                            # budget 11 -> 3 pages
    s.add(Request("c", pc, 3))                            # budget 7 -> 2 pages
    s.add(Request("d", pd, 1))                            # 1 page, but behind c: strict arrival order
    s.step()
    assert [r.id for r in s.running] == ["a", "b"] and [r.id for r in s.waiting] == ["c", "d"]
    assert s.stats.waits_for_pages >= 1
    while "b" not in s.finished:
        s.step()
        assert all(f >= 0 for f in eng.cache.free_pages())
    s.step()
    assert "c" in [r.id for r in s.running] + list(s.finished)
    done = s.run()
    for rid, prompt, n in (("a", pa, 6), ("b", pb, 5), ("c", pc, 3), ("d", pd, 1)):
        assert done[rid].output == expected_output(prompt, n), rid
    assert eng.cache.free_pages() == [6]


def test_reservation_counts_what_running_requests_may_still_claim():
    eng = FakeEngine(num_pages=5, share=False)
    s = Scheduler(eng, max_step_tokens=64, prefill_chunk=64)
    s.add(Request("a", [1, 2], 11))                       # holds 1 page now, may grow to 3
    s.step()
    s.add(Request("b", [5] * 9, 1))                       # needs 3 pages; 4 are free, but 2 are promised to a
    s.step()
    assert [r.id for r in s.waiting] == ["b"]
    done = s.run()
    assert done["a"].output == expected_output([1, 2], 11) and done["b"].output == expected_output([5] * 9, 1)


def test_known_beginnings_are_adopted():
    eng = FakeEngine(num_pages=12, share=True)
    s = Scheduler(eng)
    prompt = list(range(1, 15))
    s.add(Request("a", prompt, 2))
    s.run()
    s.add(Request("b", prompt[:10] + [40, 41], 2))
    done = s.run()
    assert s.stats.prefix_tokens_reused == 8              # two full pages of four
    assert eng.calls[-2] == [("b", 4, [3])]               # only the rest of the prompt is run
    assert done["b"].output == expected_output(prompt[:10] + [40, 41], 2)


def test_requests_that_begin_alike_wait_for_the_first_and_adopt_its_pages():
    eng = FakeEngine(num_pages=32, page_size=4, max_requests=4, share=True)
    s = Scheduler(eng, max_step_tokens=16, prefill_chunk=6)
    common = list(range(1, 22))                            # five full pages and one token
    prompts = {"a": common + [30, 31], "b": common + [40], "c": [9] + common, "d": common[:9] + [45, 46, 47]}
    for rid, prompt in prompts.items():
        s.add(Request(rid, prompt, 3))
    done = s.run()
    for rid, prompt in prompts.items():
        assert done[rid].output == expected_output(prompt, 3), rid
    # b waited until a had published the five pages they share, c (another first token) shares nothing,
    # d shares two pages
    assert s.stats.prefix_tokens_reused == 20 + 8 and s.stats.waits_for_prefix > 0
    assert s.stats.prompt_tokens == sum(len(p) for p in prompts.values()) - 28
    assert all(("b", n, w) not in call for call in eng.calls[:3] for n in range(8) for w in ([], [0]))
    assert eng.cache.free_pages() == [32]


def test_cancel_and_zero_new_tokens():
    eng = FakeEngine()
    s = Scheduler(eng)
    s.add(Request("a", [1, 2, 3], 5))
    s.add(Request("z", [1, 2, 3], 0))
    s.step()
    s.cancel("a")
    s.run()
    assert s.finished["a"].finish_reason == "cancelled" and s.finished["z"].output == []
    assert eng.cache.free_pages() == [8]


def test_temperature_requests_get_their_own_generator():
    s = Scheduler(FakeEngine())
    r = Request("a", [1], 1, SampleParams(temperature=0.8), seed=0)
    s.add(r)
    assert r.rng is not None and r.rng.state == 1         # 0 is mapped to 1


def test_a_request_id_names_one_request_at_a_time():
    """A second request under an id that is waiting, running, open in the engine or finished and not yet
    collected is refused at `add`; it never reaches admission, where it would fail on every step and
    block everyone behind it."""
    eng = FakeEngine(num_pages=16)
    sched = Scheduler(eng, max_step_tokens=8, prefill_chunk=4)
    sched.add(Request("a", [1, 2, 3], 3))
    with pytest.raises(RequestRefused):
        sched.add(Request("a", [4, 5], 2))                 # waiting
    sched.step()
    assert [r.id for r in sched.running] == ["a"]
    with pytest.raises(RequestRefused):
        sched.add(Request("a", [4, 5], 2))                 # running
    eng.cache.open("session")                              # held by someone else, a session for instance
    with pytest.raises(RequestRefused):
        sched.add(Request("session", [4, 5], 2))
    sched.add(Request("b", [4, 5], 2))                     # the queue is not blocked by the refusals
    done = sched.run()
    assert done["a"].output == expected_output([1, 2, 3], 3) and done["b"].output == expected_output([4, 5], 2)
    with pytest.raises(RequestRefused):
        sched.add(Request("a", [9], 1))                    # finished, its result not collected yet
    first = sched.finished.pop("a")
    sched.add(Request("a", [9], 1))
    assert sched.run()["a"] is not first and sched.finished["a"].output == expected_output([9], 1)
    assert sched.stats.refused == 4
    eng.cache.close("session")
    eng.cache.check()


class FailingEngine(FakeEngine):
    """The step function raises on the calls named in `fail_on` (1-based), after it has undone what it
    reserved for that step, as the real engine does."""

    def __init__(self, fail_on, **kw):
        super().__init__(**kw)
        self.fail_on = set(fail_on)
        self.tries = 0

    def step(self, entries, borrow=False):
        self.tries += 1
        if self.tries in self.fail_on:
            reqs, opened = [], []
            for e in entries:
                if e.request not in self.cache.requests:
                    self.cache.open(e.request)
                    opened.append(e.request)
                reqs.append(self.cache.requests[e.request])
            self.cache.reserve([(r, len(e.tokens)) for r, e in zip(reqs, entries)])
            for r in reqs:
                self.cache.trim(r)
            for rid in opened:
                self.cache.close(rid)
            raise RuntimeError("the device said no")
        return super().step(entries, borrow)


def test_a_failed_step_fails_its_requests_and_the_queue_moves_on():
    """/root/reference/src/kipp_server.c:2081-2088: the batch fails as a unit.  Requests that had tokens in
    the failed step end as failed and give everything back; a request that waited is admitted and runs."""
    eng = FailingEngine(fail_on=[3], num_pages=6, page_size=4)
    sched = Scheduler(eng, max_step_tokens=8, prefill_chunk=4)
    sched.add(Request("a", list(range(1, 9)), 4))          # 11 tokens: 3 pages
    sched.add(Request("b", [7, 8, 9], 6))                  # 8 tokens: 2 pages
    sched.add(Request("c", [4, 5, 6, 7, 8], 8))            # 12 tokens: 3 pages, waits until a or b has gone
    done = sched.run(max_steps=50)
    assert sched.idle
    assert done["a"].finish_reason == "failed" and done["b"].finish_reason == "failed"
    assert "the device said no" in done["a"].error and done["a"].error == done["b"].error
    assert done["c"].finish_reason == "length" and done["c"].output == expected_output([4, 5, 6, 7, 8], 8)
    st = sched.stats
    assert (st.failed, st.failed_steps, st.finished, st.requests) == (2, 1, 3, 3)
    assert st.queue_wait_count == 3 and st.queue_wait_seconds_sum >= 0.0
    assert st.ttft_count >= 1 and st.ttft_seconds_sum >= 0.0 and st.decode_seconds_sum >= 0.0
    assert not eng.cache.requests and eng.cache.free_pages() == [6]
    eng.cache.check()


def test_a_failed_step_leaves_requests_outside_it_running():
    """With a budget of one token a step, the step that fails holds one request only; the other goes on
    and produces what it would have produced."""
    eng = FailingEngine(fail_on=[4], num_pages=8, page_size=4)
    sched = Scheduler(eng, max_step_tokens=1, prefill_chunk=4)
    sched.add(Request("a", [1, 2], 3))
    sched.add(Request("b", [3, 4], 3))
    done = sched.run(max_steps=60)
    reasons = sorted(r.finish_reason for r in done.values())
    assert reasons == ["failed", "length"]
    ok = [r for r in done.values() if r.finish_reason == "length"][0]
    assert ok.output == expected_output(list(ok.prompt), 3)
    assert sched.stats.failed == 1 and eng.cache.free_pages() == [8]
    eng.cache.check()


def test_a_windowed_group_with_a_small_pool_of_its_own():
    """A model whose second run keeps a window of 6 keys in pages of 2: its pool is sized for the windows of the
    running requests, not for their whole contexts, and admission counts what each may still hold there."""
    class TwoGroups(FakeEngine):
        def __init__(self):
            self.cache = CacheManager([KVNeed(1, 16), KVNeed(1, 16, window=6, page_size=2)], [None, None], 4, [24, 14],
                                      max_requests=4, max_position=64, runtime=None, share_prefixes=False)
            self.vocab_size = VOCAB
            self.calls = []
    eng = TwoGroups()
    sched = Scheduler(eng, max_step_tokens=8, prefill_chunk=4)
    # a request holds at most the pages of 6 - 1 + 4 tokens and one more in the windowed group: 6 of 14, so two run and a third waits
    for name, prompt in (("a", list(range(1, 21))), ("b", list(range(2, 19))), ("c", [5, 6, 7])):
        sched.add(Request(name, prompt, 12))
    sched.step()
    assert [r.id for r in sched.running] == ["a", "b"] and [r.id for r in sched.waiting] == ["c"]
    done = sched.run(max_steps=200)
    for name, prompt in (("a", list(range(1, 21))), ("b", list(range(2, 19))), ("c", [5, 6, 7])):
        assert done[name].output == expected_output(prompt, 12)
    assert eng.cache.free_pages() == [24, 14] and sched.stats.waits_for_pages > 0
    with pytest.raises(RequestRefused):
        big = Scheduler(eng, max_step_tokens=64, prefill_chunk=32)      # steps of 32 tokens: 19 pages of 2 at once
        big.add(Request("d", list(range(40)), 2))
    eng.cache.check()
