"""The scheduler's decisions, on the CPU, with the real cache manager and a stand-in for the model
(the next token is a function of the tokens so far, so recomputation after a preemption must give
the same output as an undisturbed run)."""
import pytest
import torch

from tlie_amd import EngineError, ErrorCode
from tlie_amd.cache import CacheManager, RunNeed
from tlie_amd.engine import Request, SamplingParams, Scheduler
from tlie_amd.parts import CacheNeed


def make(num_pages=16, page_size=4, max_requests=4, **kwargs):
    cache = CacheManager([RunNeed(0, CacheNeed((2, 1), 8))], page_size, num_pages, max_requests, torch.float32, "cpu",
                         max_positions=kwargs.pop("max_positions", 64))
    return cache, Scheduler(cache, max_positions=cache.max_positions, **kwargs)


def fake_token(tokens):
    return (sum(tokens) * 31 + len(tokens) * 7) % 97


def drive(cache, scheduler, log=None, max_steps=500, finish=True):
    """Runs plans against the cache manager as the engine loop does, to the end (or, with
    finish=False, for max_steps steps)."""
    for _ in range(max_steps):
        if not scheduler.has_work():
            return
        plan = scheduler.schedule()
        assert plan, "no progress"
        seen = set()
        for item in plan:
            assert item.request.id not in seen
            seen.add(item.request.id)
            assert item.first == cache.length(item.request.id) == item.request.computed
        assert cache.can_reserve([(item.request.id, item.count) for item in plan])
        for item in plan:
            cache.reserve(item.request.id, item.count)
            cache.commit(item.request.id, item.count)
        if log is not None:
            log.append([(item.request.id, item.first, item.count, item.samples) for item in plan])
        sampled = [fake_token(item.request.tokens[:item.first + item.count]) for item in plan if item.samples]
        scheduler.update(plan, sampled)
        cache.check()
    if finish:
        raise AssertionError("did not finish")


def expected_output(prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        out.append(fake_token(tokens))
        tokens.append(out[-1])
    return out


def test_prompt_is_cut_under_the_budget_then_decodes():
    cache, scheduler = make(max_tokens_per_step=8)
    request = Request("a", list(range(1, 20)), SamplingParams(max_tokens=3))
    scheduler.add(request)
    log = []
    drive(cache, scheduler, log)
    assert log == [[("a", 0, 8, False)], [("a", 8, 8, False)], [("a", 16, 3, True)], [("a", 19, 1, True)], [("a", 20, 1, True)]]
    assert request.generated == expected_output(request.prompt, 3) and request.finish_reason == "length"
    assert cache.free_pages() == [16] and cache.free_slots == 4       # everything came back
    # the last sampled token is never fed back (app/reference_cli.cpp:103): 19 + 2 positions were cached
    assert scheduler.stats["prefill_tokens"] == 19 and scheduler.stats["decode_tokens"] == 2


def test_decodes_first_then_fills_with_prompt_portions_fifo():
    cache, scheduler = make(max_tokens_per_step=6, num_pages=32)
    a = Request("a", [1, 2, 3], SamplingParams(max_tokens=4))
    b = Request("b", list(range(10, 21)), SamplingParams(max_tokens=2))
    c = Request("c", [5, 6], SamplingParams(max_tokens=2))
    for request in (a, b, c):
        scheduler.add(request)
    log = []
    drive(cache, scheduler, log)
    assert log[0] == [("a", 0, 3, True), ("b", 0, 3, False)]            # first come first served under 6 tokens
    assert log[1] == [("a", 3, 1, True), ("b", 3, 5, False)]            # the decoding request comes first
    assert log[2] == [("a", 4, 1, True), ("b", 8, 3, True), ("c", 0, 2, True)]
    for request in (a, b, c):
        assert request.generated == expected_output(request.prompt, request.params.max_tokens)


def test_prompts_beside_decoding_requests_can_be_capped():
    """A step's time grows with its prompt tokens and its decoding requests wait for all of it: with
    a cap, prompts get at most so many tokens in a step that also decodes, and the whole budget in a
    step that does not.  The outputs do not change."""
    def run(cap):
        cache, scheduler = make(max_tokens_per_step=16, num_pages=32, prompt_tokens_beside_decodes=cap)
        a = Request("a", [1, 2, 3], SamplingParams(max_tokens=6))
        b = Request("b", list(range(10, 40)), SamplingParams(max_tokens=2))
        scheduler.add(a)
        log = []
        drive(cache, scheduler, log, max_steps=1, finish=False)     # "a" is decoding when "b" arrives
        scheduler.add(b)
        drive(cache, scheduler, log)
        assert a.generated == expected_output(a.prompt, 6) and b.generated == expected_output(b.prompt, 2)
        return log
    free = run(None)
    assert free[1] == [("a", 3, 1, True), ("b", 0, 15, False)] and free[2] == [("a", 4, 1, True), ("b", 15, 15, True)]
    capped = run(4)
    assert capped[1] == [("a", 3, 1, True), ("b", 0, 4, False)] and capped[2] == [("a", 4, 1, True), ("b", 4, 4, False)]
    # once "a" has finished (its fifth decode step is the trace's sixth), the prompt takes the whole budget again
    alone = [step for step in capped if [item[0] for item in step] == ["b"]]
    assert alone and alone[0][0][2] == 10                      # the 10 tokens that were left, in one step
    with pytest.raises(EngineError):
        make(prompt_tokens_beside_decodes=0)


def test_admission_waits_for_a_slot():
    cache, scheduler = make(max_requests=2, num_pages=32)
    requests = [Request(i, [i + 1, i + 2], SamplingParams(max_tokens=3)) for i in range(4)]
    for request in requests:
        scheduler.add(request)
    log = []
    drive(cache, scheduler, log)
    assert [entry[0] for entry in log[0]] == [0, 1]
    first_of = {rid: index for index, step in enumerate(log) for (rid, first, _, _) in step if first == 0}
    assert first_of[2] == 3 and first_of[3] == 3                          # after the first two finished (3 outputs)
    for request in requests:
        assert request.generated == expected_output(request.prompt, 3)


def test_requests_that_can_never_fit_are_refused():
    cache, scheduler = make(num_pages=4, page_size=4, max_positions=64)
    with pytest.raises(EngineError) as caught:
        scheduler.add(Request("big", list(range(1, 17)), SamplingParams(max_tokens=2)))     # needs 17 positions, pool holds 16
    assert caught.value.code == ErrorCode.OUT_OF_MEMORY
    scheduler.add(Request("fits", list(range(1, 16)), SamplingParams(max_tokens=2)))         # 16 positions
    with pytest.raises(EngineError) as caught:
        scheduler.add(Request("long", list(range(60)), SamplingParams(max_tokens=5)))
    assert caught.value.code == ErrorCode.OUT_OF_BOUNDS                   # app/reference_cli.cpp:72-75
    with pytest.raises(EngineError):
        scheduler.add(Request("empty", [], SamplingParams(max_tokens=5)))
    with pytest.raises(EngineError):
        scheduler.add(Request("zero", [1], SamplingParams(max_tokens=0)))
    with pytest.raises(EngineError):
        scheduler.add(Request("p", [1], SamplingParams(top_p=0.0)))
    drive(cache, scheduler)


def test_pages_run_out_while_decoding_the_last_admitted_is_preempted():
    # 6 pages of 4: two requests of 9-token prompts take 3 pages each (positions 0..11); when they
    # grow past 12 positions each needs a fourth page and none is free.  (Admitted as soon as a first
    # portion fits: by default the second would wait for the first to finish, see below.)
    cache, scheduler = make(num_pages=6, page_size=4, admit_partial=True)
    a = Request("a", list(range(1, 10)), SamplingParams(max_tokens=8))
    b = Request("b", list(range(21, 30)), SamplingParams(max_tokens=8))
    scheduler.add(a)
    scheduler.add(b)
    log = []
    drive(cache, scheduler, log)
    assert scheduler.stats["preemptions"] >= 1 and b.preemptions >= 1 and a.preemptions == 0   # the victim is the last admitted
    assert a.generated == expected_output(a.prompt, 8) and b.generated == expected_output(b.prompt, 8)
    # "b" was recomputed from position 0, its prompt and what it had generated so far: in all it ran
    # more tokens than an undisturbed run of 9 + 7
    restarts = [index for index, step in enumerate(log) if index > 0 for (rid, first, _, _) in step if rid == "b" and first == 0]
    assert restarts
    assert sum(count for step in log for (rid, _, count, _) in step if rid == "b") > 16
    assert sum(count for step in log for (rid, _, count, _) in step if rid == "a") == 16
    assert cache.free_pages() == [6] and cache.free_slots == 4


def test_a_preempted_request_returns_its_tokens_to_the_steps_budget():
    """Three decoding requests under a budget of 3 tokens, the last admitted also the first in this
    step's rotation: when the second one finds no page and preempts it, the token it had in the plan is
    free again, so the step still takes the other two (the budget is not charged for a request that
    left the plan)."""
    cache, scheduler = make(num_pages=6, page_size=4, max_tokens_per_step=3, admit_partial=True)
    requests = [Request(name, list(range(base, base + 7)), SamplingParams(max_tokens=8))
                for name, base in (("a", 1), ("b", 11), ("c", 21))]
    for request in requests:
        scheduler.add(request)
    log = []
    drive(cache, scheduler, log)
    for request in requests:
        assert request.generated == expected_output(request.prompt, 8)
    assert scheduler.stats["preemptions"] >= 1
    # in the step that preempted, what was planned never exceeded the budget, and no step of
    # several decoding requests shrank to fewer tokens than the requests that stayed could use
    for step in log:
        assert sum(count for (_, _, count, _) in step) <= 3
    assert cache.free_pages() == [6] and cache.free_slots == 4


def test_budget_after_preemption_is_what_the_plan_holds():
    """Directly: the tokens of an item that preemption takes out of the plan are handed back."""
    cache, scheduler = make(num_pages=8, page_size=4)
    a = Request("a", [1, 2, 3], SamplingParams(max_tokens=4))
    scheduler.add(a)
    plan = scheduler.schedule()
    assert [(item.request.id, item.count) for item in plan] == [("a", 3)]
    planned = [cache.pages_needed("a", 3)[0]]
    assert scheduler._preempt(a, plan, planned) == 3 and plan == [] and planned == [0]
    assert a.state == "waiting" and not cache.is_live("a")


def test_prompts_that_block_each_other_are_untangled():
    # two prompts of 28 tokens (7 pages each) in a pool of 10: cut into portions of 8 they take
    # pages turn by turn until neither can go on; the later one is preempted, the earlier finishes.
    cache, scheduler = make(num_pages=10, page_size=4, max_tokens_per_step=16, chunk_size=8, admit_partial=True)
    a = Request("a", list(range(1, 29)), SamplingParams(max_tokens=2))
    b = Request("b", list(range(31, 59)), SamplingParams(max_tokens=2))
    scheduler.add(a)
    scheduler.add(b)
    drive(cache, scheduler)
    assert a.generated == expected_output(a.prompt, 2) and b.generated == expected_output(b.prompt, 2)
    assert b.preemptions >= 1 and a.preemptions == 0


def test_a_waiting_request_is_admitted_when_all_it_brings_fits():
    # the same two prompts of 7 pages each in a pool of 10: by default the second is not admitted for a
    # first portion that would then fight the first for pages; it waits until the first has finished
    cache, scheduler = make(num_pages=10, page_size=4, max_tokens_per_step=16, chunk_size=8)
    a = Request("a", list(range(1, 29)), SamplingParams(max_tokens=2))
    b = Request("b", list(range(31, 59)), SamplingParams(max_tokens=2))
    scheduler.add(a)
    scheduler.add(b)
    log = []
    drive(cache, scheduler, log)
    assert a.generated == expected_output(a.prompt, 2) and b.generated == expected_output(b.prompt, 2)
    assert scheduler.stats["preemptions"] == 0
    last_of_a = max(index for index, step in enumerate(log) if any(rid == "a" for rid, _, _, _ in step))
    first_of_b = min(index for index, step in enumerate(log) if any(rid == "b" for rid, _, _, _ in step))
    assert first_of_b > last_of_a
    # with room for both (7 + 7 pages, a page of growth each and one to spare) they run side by side
    cache, scheduler = make(num_pages=17, page_size=4, max_tokens_per_step=16, chunk_size=8)
    a = Request("a", list(range(1, 29)), SamplingParams(max_tokens=2))
    b = Request("b", list(range(31, 59)), SamplingParams(max_tokens=2))
    scheduler.add(a)
    scheduler.add(b)
    log = []
    drive(cache, scheduler, log)
    assert any({rid for rid, _, _, _ in step} == {"a", "b"} for step in log) and scheduler.stats["preemptions"] == 0
    # a request alone is admitted whatever it needs (`add` has refused what the pool could never hold)
    cache, scheduler = make(num_pages=8, page_size=4)
    alone = Request("x", list(range(1, 29)), SamplingParams(max_tokens=4))
    scheduler.add(alone)
    drive(cache, scheduler)
    assert alone.generated == expected_output(alone.prompt, 4)


def test_requests_that_outnumber_the_pool_many_times():
    """Twenty requests of 21 to 40 prompt tokens and 12 outputs on a pool of 30 pages of 4 (three of
    them at a time): the outputs are those of undisturbed runs under either way of admitting; admitted
    whole, requests are preempted only when those that run outgrow the page of growth kept for each, a
    fraction of what admitting first portions costs."""
    counts = {}
    for partial in (False, True):
        cache, scheduler = make(num_pages=30, page_size=4, max_requests=8, max_tokens_per_step=32, admit_partial=partial)
        requests = [Request(f"r{i}", [(7 * i + j) % 50 + 1 for j in range(21 + i)], SamplingParams(max_tokens=12)) for i in range(20)]
        for request in requests:
            scheduler.add(request)
        drive(cache, scheduler, max_steps=5000)
        for request in requests:
            assert request.generated == expected_output(request.prompt, 12)
        assert cache.free_pages() == [30] and cache.free_slots == 8
        counts[partial] = (scheduler.stats["preemptions"], scheduler.stats["prefill_tokens"])
    assert counts[True][0] >= 10 and counts[False][0] * 3 <= counts[True][0], counts
    assert counts[False][1] < counts[True][1]              # and fewer prompt tokens run twice


def test_more_decoders_than_the_budget_rotate():
    cache, scheduler = make(num_pages=32, max_requests=4, max_seqs_per_step=2, max_tokens_per_step=64)
    requests = [Request(i, [i + 1], SamplingParams(max_tokens=5)) for i in range(4)]
    for request in requests:
        scheduler.add(request)
    log = []
    drive(cache, scheduler, log)
    assert all(len(step) <= 2 for step in log)
    for request in requests:
        assert request.generated == expected_output(request.prompt, 5)       # nobody starves


def test_abort_and_eos():
    cache, scheduler = make()
    a = Request("a", [1, 2, 3], SamplingParams(max_tokens=50))
    scheduler.add(a)
    scheduler.update(plan := scheduler.schedule(), [fake_token(a.prompt)])
    for item in plan:
        pass
    assert scheduler.abort("a") and a.finish_reason == "aborted" and not scheduler.has_work()
    assert not scheduler.abort("a")
    cache2, scheduler2 = make(eos_token_id=fake_token([4, 5]))
    b = Request("b", [4, 5], SamplingParams(max_tokens=50, stop_on_eos=True))
    scheduler2.add(b)
    drive(cache2, scheduler2)
    assert b.finish_reason == "eos" and len(b.generated) == 1


def drive_a_step_behind(cache, scheduler, max_steps=500):
    """As the engine loop runs when the host is one step behind the device: a step's tokens are
    written into the requests only after the next step has been planned and 'launched'; plans that
    need a token earlier (a recomputation after a preemption) get it first.  Returns how many
    steps were planned without the tokens of the step before."""
    behind, ahead = None, 0

    def settle():
        nonlocal behind
        if behind is not None:
            scheduler.resolve(*behind)
            behind = None

    for _ in range(max_steps):
        if not scheduler.has_work():
            settle()
            return ahead
        plan = scheduler.schedule()
        assert plan, "no progress"
        for item in plan:
            request = item.request
            if request.pending and item.first + item.count == request.total and item.count != 1:
                settle()                                   # a recomputed portion reaches the pending token
        ahead += behind is not None
        for item in plan:
            cache.reserve(item.request.id, item.count)
            cache.commit(item.request.id, item.count)
        known = behind
        settle()                                           # "while the step runs"
        sampled = [fake_token(item.request.token_slice(0, item.first + item.count)) for item in plan if item.samples]
        assert known is None or all(token >= 0 for item in plan for token in item.request.token_slice(0, item.first + item.count))
        if scheduler.can_defer(plan):
            scheduler.update(plan, None)
            behind = (plan, sampled)
        else:
            scheduler.update(plan, sampled)
        cache.check()
    if finish:
        raise AssertionError("did not finish")


def test_tokens_may_arrive_a_step_late():
    from tlie_amd.engine.scheduler import PENDING
    # ample pages: every decode step is planned before the last one's tokens are in
    cache, scheduler = make(num_pages=32, max_tokens_per_step=8, chunk_size=4)
    requests = [Request(name, list(range(3 + 2 * i, 9 + 3 * i)), SamplingParams(max_tokens=7 + i)) for i, name in enumerate("abc")]
    for request in requests:
        scheduler.add(request)
    ahead = drive_a_step_behind(cache, scheduler)
    assert ahead > 10
    for request in requests:
        assert request.generated == expected_output(request.prompt, request.params.max_tokens) and request.finish_reason == "length"
    # few pages: preemptions recompute prompts that end in a token still pending; the output is the same
    cache, scheduler = make(num_pages=7, max_tokens_per_step=16)
    requests = [Request(name, [i + 1, i + 2, i + 3, i + 4, i + 5], SamplingParams(max_tokens=12)) for i, name in enumerate("abc")]
    for request in requests:
        scheduler.add(request)
    drive_a_step_behind(cache, scheduler)
    assert scheduler.stats["preemptions"] > 0
    for request in requests:
        assert request.generated == expected_output(request.prompt, 12)
    # a request that stops at the end-of-sequence token cannot wait for its tokens
    eos = expected_output([4, 5], 3)[2]
    cache, scheduler = make(eos_token_id=eos)
    stopper = Request("s", [4, 5], SamplingParams(max_tokens=50, stop_on_eos=True))
    other = Request("o", [9, 9, 9], SamplingParams(max_tokens=6))
    scheduler.add(stopper)
    scheduler.add(other)
    drive_a_step_behind(cache, scheduler)
    assert stopper.finish_reason == "eos" and stopper.generated == expected_output([4, 5], 3)
    assert other.generated == expected_output([9, 9, 9], 6)
    # resolve refuses what update did not leave pending
    cache, scheduler = make()
    request = Request("r", [1, 2], SamplingParams(max_tokens=3))
    scheduler.add(request)
    plan = scheduler.schedule()
    scheduler.update(plan, None)
    assert request.generated == [PENDING] and request.pending
    scheduler.resolve(plan, [55])
    assert request.generated == [55] and not request.pending
    with pytest.raises(EngineError):
        scheduler.resolve(plan, [56])


def test_token_slice_is_the_slice_of_prompt_and_generated():
    request = Request("r", [10, 11, 12, 13], SamplingParams(max_tokens=9), generated=[20, 21, 22])
    for first in range(7):
        for count in range(0, 8 - first):
            assert request.token_slice(first, count) == request.tokens[first:first + count]
    assert request.total == 7
