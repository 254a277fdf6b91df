"""The scheduler's decisions, on the host with a fake executor.  Vectors and
invariants follow the reference's tests/unit/scheduler_test.cc (lines cited per test)."""
import pytest

from inferx_amd.cache.manager import CacheManager, GroupLayout
from inferx_amd.engine.batch import build_step_batch
from inferx_amd.engine.scheduler import (FINISH_CANCELLED, FINISH_CONTEXT, FINISH_LENGTH, FINISH_OOM, FINISH_STOP,
                                         Scheduler)
from inferx_amd.sampling import SamplingParams


def make(pages=64, page_size=4, max_running=8, budget=2048, max_seq_len=None, groups=None):
    groups = groups or [GroupLayout(0)]
    cache = CacheManager(groups, [pages] * len(groups), page_size, max_running, max_seq_len or pages * page_size)
    return Scheduler(cache, max_running, budget, max_seq_len), cache


def P(n, **kw):
    return SamplingParams(max_tokens=n, **kw)


def fake_token(position):
    return 100 + (position * 7) % 50  # a function of the position only (scheduler_test.cc:700-731)


def drain(sched, cache, max_steps=4000, check=None):
    done = []
    for _ in range(max_steps):
        if not sched.has_work():
            break
        plan = sched.prepare_step()
        if plan is not None:
            batch = build_step_batch(cache, plan.entries())
            batch.validate(10 ** 6, [p.num_pages for p in cache.pools], cache.page_size)  # every slot under its table
            if check:
                check(plan, batch)
            sched.commit_step([fake_token(int(batch.positions[r])) for r in batch.logits_rows])
        done += sched.take_completed()
        cache.check()
    return done + sched.take_completed()


def test_first_step_is_the_whole_prompt_with_one_logits_row():
    # scheduler_test.cc:93-114
    sched, cache = make()
    sched.add_request(1, [10, 11, 12, 13, 14], P(3))
    plan = sched.prepare_step()
    batch = build_step_batch(cache, plan.entries())
    assert batch.token_ids.tolist() == [10, 11, 12, 13, 14]
    assert batch.positions.tolist() == [0, 1, 2, 3, 4]
    assert batch.logits_rows.tolist() == [4]
    assert cache.pools[0].used_pages == 2  # 5 tokens, pages of 4
    # slots cross the page boundary (scheduler_test.cc:149-166)
    row = cache.block_row(1, 0)
    assert batch.slots[0].tolist() == [row[0] * 4 + i for i in range(4)] + [row[1] * 4]


def test_budget_remainder_is_a_portion():
    # scheduler_test.cc:425-446
    sched, cache = make(budget=4)
    sched.add_request(1, [1, 2, 3], P(2))
    sched.add_request(2, [4, 5, 6], P(2))
    batch = build_step_batch(cache, sched.prepare_step().entries())
    assert batch.token_ids.tolist() == [1, 2, 3, 4]
    assert batch.seq_of_token.tolist() == [0, 0, 0, 1]
    assert batch.positions.tolist() == [0, 1, 2, 0]
    assert batch.logits_rows.tolist() == [2]
    assert batch.seq_lens.tolist() == [3, 1]


def test_decodes_before_prompt_portions():
    # scheduler_test.cc:505-532
    sched, cache = make(budget=4)
    sched.add_request(1, [1, 2], P(10))
    plan = sched.prepare_step()
    assert plan.num_tokens == 2
    sched.commit_step([50])
    sched.add_request(2, [7] * 8, P(1))
    batch = build_step_batch(cache, sched.prepare_step().entries())
    assert batch.seq_of_token.tolist() == [0, 1, 1, 1]
    assert batch.token_ids.tolist() == [50, 7, 7, 7]
    assert batch.logits_rows.tolist() == [0]
    assert batch.seq_lens.tolist() == [3, 3]


def test_long_prompt_runs_in_portions_every_position_once():
    # scheduler_test.cc:451-501: 15 tokens at budget 4 = 4 portions
    sched, cache = make(budget=4)
    sched.add_request(1, list(range(15)), P(1))
    seen, portions = [], []

    def check(plan, batch):
        seen.extend(batch.positions.tolist())
        portions.append(plan.num_tokens)
        # a middle portion asks for no logits (scheduler_test.cc:579-590)
        assert len(batch.logits_rows) == (1 if seen[-1] == 14 else 0)

    done = drain(sched, cache, check=check)
    assert portions == [4, 4, 4, 3] and seen == list(range(15))
    assert done[0].reason == FINISH_LENGTH and len(done[0].output_tokens) == 1


def test_portions_change_steps_not_work():
    # scheduler_test.cc:537-575: same (token, position) pairs whatever the budget
    def work(budget):
        sched, cache = make(budget=budget)
        sched.add_request(1, list(range(40, 53)), P(4))
        pairs = []
        out = drain(sched, cache, check=lambda plan, b: pairs.extend(zip(b.token_ids.tolist(), b.positions.tolist())))
        return pairs, out[0].output_tokens

    assert work(3) == work(2048)


def test_stop_token_is_kept_and_pages_come_back():
    # scheduler_test.cc:168-190, 210-228
    sched, cache = make()
    sched.add_request(1, [1, 2, 3], P(10, stop_tokens=[fake_token(3)]))
    done = drain(sched, cache)
    assert done[0].reason == FINISH_STOP and done[0].output_tokens == [fake_token(2), fake_token(3)]
    assert cache.pools[0].used_pages == 0 and not cache.live_requests()


def test_fcfs_and_deferral_without_leak():
    # scheduler_test.cc:267-287, 364-400: the second prompt does not fit beside the first and waits
    sched, cache = make(pages=4, page_size=4)
    sched.add_request(1, list(range(12)), P(2))
    sched.add_request(2, list(range(8)), P(2))
    plan = sched.prepare_step()
    assert [c.rid for c in plan.contributions] == [1] and len(sched.waiting) == 1
    assert cache.pools[0].used_pages == 3 and cache.live_requests() == [1]
    sched.commit_step([5])
    done = drain(sched, cache)
    assert [c.rid for c in done] == [1, 2] and cache.pools[0].used_pages == 0


def test_context_limit_retires_only_that_sequence():
    # scheduler_test.cc:903-959: 16-token context, 2-token prompt -> 15 generated tokens
    sched, cache = make(pages=64, page_size=4, max_seq_len=16)
    sched.add_request(1, [1, 2], P(100))
    sched.add_request(2, [3, 4], P(3))
    done = {c.rid: c for c in drain(sched, cache)}
    assert done[1].reason == FINISH_CONTEXT and len(done[1].output_tokens) == 15
    assert done[2].reason == FINISH_LENGTH and len(done[2].output_tokens) == 3


def test_lone_sequence_runs_out_of_pages():
    # scheduler_test.cc:963-984: 3 pages of 4, 2-token prompt -> 11 generated tokens, then out_of_memory
    sched, cache = make(pages=3, page_size=4, max_seq_len=64)
    sched.add_request(1, [1, 2], P(100))
    done = drain(sched, cache)
    assert done[0].reason == FINISH_OOM and len(done[0].output_tokens) == 11
    assert cache.pools[0].used_pages == 0


def test_prompt_larger_than_the_pool_ends_instead_of_waiting_for_ever():
    # 2 pages of 4 and a prompt of 20: nothing runs, so nobody will ever give a page back.  The request ends
    # out_of_memory at once, nothing is held, and the request behind it runs (the reference's "retires rather
    # than spinning", scheduler_test.cc:963-984, at admission)
    sched, cache = make(pages=2, page_size=4, max_seq_len=64)
    sched.add_request("a", list(range(20)), P(4))
    sched.add_request("b", [1, 2, 3], P(2))
    plan = sched.prepare_step()
    early = sched.take_completed()
    assert [(c.rid, c.reason, c.output_tokens) for c in early] == [("a", FINISH_OOM, [])]
    assert plan is not None and [e[0] for e in plan.entries()] == ["b"]
    batch = build_step_batch(cache, plan.entries())
    sched.commit_step([fake_token(int(batch.positions[r])) for r in batch.logits_rows])
    done = drain(sched, cache)
    assert [(c.rid, c.reason, len(c.output_tokens)) for c in done] == [("b", FINISH_LENGTH, 2)]
    assert cache.pools[0].used_pages == 0 and not sched.has_work()
    cache.check()


def test_large_prompt_behind_a_running_one_waits_then_ends():
    # while something runs, a prompt that does not fit waits at the head (pages may come back); once the pool is
    # all free and it still does not fit, it ends
    sched, cache = make(pages=3, page_size=4, max_seq_len=64)
    sched.add_request("small", [1, 2], P(3))
    sched.add_request("big", list(range(16)), P(1))
    done = drain(sched, cache, max_steps=50)
    assert [(c.rid, c.reason) for c in done] == [("small", FINISH_LENGTH), ("big", FINISH_OOM)]
    assert not sched.has_work() and cache.pools[0].used_pages == 0


def test_abandoned_step_is_planned_again():
    # a step whose launch failed is dropped and the same work is planned afresh, nothing lost or counted twice
    sched, cache = make(budget=4)
    sched.add_request(1, [1, 2, 3, 4, 5, 6], P(2))
    first = sched.prepare_step().entries()
    with pytest.raises(RuntimeError, match="twice"):
        sched.prepare_step()
    sched.abandon_step()
    assert sched.prepare_step().entries() == first
    sched.abandon_step()
    done = drain(sched, cache)
    assert done[0].reason == FINISH_LENGTH and len(done[0].output_tokens) == 2
    assert cache.pools[0].used_pages == 0


def test_prompt_longer_than_the_context_is_refused():
    sched, cache = make(max_seq_len=8)
    sched.add_request(1, list(range(9)), P(1))
    done = drain(sched, cache)
    assert done[0].reason == FINISH_OOM and done[0].output_tokens == []


def test_preempted_output_equals_unpreempted():
    # scheduler_test.cc:742-812, 817-895
    def run(pages):
        sched, cache = make(pages=pages, page_size=4, max_seq_len=64)
        sched.add_request(1, [1, 2, 3], P(12))
        sched.add_request(2, [4, 5, 6, 7], P(12))
        sched.add_request(3, [8, 9], P(12))
        out = {c.rid: (c.output_tokens, c.reason) for c in drain(sched, cache)}
        return out, sched.preemptions

    roomy, n0 = run(64)
    tight, n1 = run(7)
    assert n0 == 0 and n1 > 0
    assert roomy == tight
    assert all(reason == FINISH_LENGTH for _, reason in tight.values())


def test_newest_is_preempted_and_waits_at_the_head():
    sched, cache = make(pages=4, page_size=4, max_seq_len=64)
    sched.add_request(1, [1, 2, 3, 4, 5, 6, 7], P(20))   # two pages
    sched.add_request(2, [1, 2, 3, 4, 5, 6, 7], P(20))   # two pages: the pool is full
    sched.add_request(3, [9], P(1))
    sched.commit_step([5, 5]) if sched.prepare_step() else None
    # both want their 9th slot next step but one: request 1 grows first, request 2 (newest) gives way
    steps = 0
    while sched.preemptions == 0 and steps < 10:
        plan = sched.prepare_step()
        sched.commit_step([5] * sum(c.samples for c in plan.contributions))
        steps += 1
    assert sched.preemptions == 1
    assert [s.rid for s in sched.running] == [1] and sched.waiting[0].rid == 2 and sched.waiting[1].rid == 3
    cache.check()


def test_cancel():
    sched, cache = make()
    sched.add_request(1, [1, 2, 3], P(50))
    sched.add_request(2, [1, 2, 3], P(2))
    sched.commit_step([7, 7]) if sched.prepare_step() else None
    sched.cancel(1)
    done = {c.rid: c for c in drain(sched, cache)}
    assert done[1].reason == FINISH_CANCELLED and done[1].output_tokens == [7]
    assert done[2].reason == FINISH_LENGTH and cache.pools[0].used_pages == 0


def test_wrong_count_commit_is_an_error():
    sched, cache = make()
    sched.add_request(1, [1, 2, 3], P(5))
    sched.prepare_step()
    with pytest.raises(ValueError):
        sched.commit_step([1, 2])


def test_max_running_and_windowed_group():
    sched, cache = make(pages=12, page_size=4, max_running=2, max_seq_len=48, groups=[GroupLayout(0), GroupLayout(6)])
    for rid in range(4):
        sched.add_request(rid, list(range(5 + rid)), P(20))
    live = []
    done = drain(sched, cache, check=lambda plan, b: live.append(len(plan.contributions)))
    assert max(live) <= 2 and len(done) == 4 and all(c.reason == FINISH_LENGTH for c in done)
    assert all(p.used_pages == 0 for p in cache.pools)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_arrivals_scarce_pages(seed):
    """Requests arrive at random steps, some are cancelled, pages are scarce so that sequences are preempted:
    every request finishes exactly once, no page or slot is lost at any step, every step keeps its budget, and
    (tokens being a function of the position) each output equals the one of an unconstrained run."""
    import random
    rng = random.Random(seed)
    n_req = 14
    prompts = {r: [rng.randrange(1000) for _ in range(rng.randrange(1, 40))] for r in range(n_req)}
    limits = {r: rng.randrange(1, 30) for r in range(n_req)}
    arrive = {r: rng.randrange(0, 25) for r in range(n_req)}
    cancel_at = {r: arrive[r] + rng.randrange(0, 12) for r in rng.sample(range(n_req), 3)}

    def run(pages, budget, cancels):
        sched, cache = make(pages=pages, page_size=4, max_running=4, budget=budget, max_seq_len=80)
        done, step = [], 0
        while step < 60 or sched.has_work():
            for r in range(n_req):
                if arrive[r] == step:
                    sched.add_request(r, prompts[r], P(limits[r]))
                if cancels and cancel_at.get(r) == step:
                    sched.cancel(r)
            plan = sched.prepare_step()
            if plan is not None:
                assert 0 < plan.num_tokens <= budget and len(plan.contributions) <= 4
                batch = build_step_batch(cache, plan.entries())
                batch.validate(10 ** 6, [p.num_pages for p in cache.pools], cache.page_size)
                sched.commit_step([fake_token(int(batch.positions[r])) for r in batch.logits_rows])
            done += sched.take_completed()
            cache.check()
            step += 1
            assert step < 5000
        assert all(p.used_pages == 0 for p in cache.pools) and not cache.live_requests()
        return {c.rid: c for c in done}, sched.preemptions, len(done)

    free, _, n_free = run(pages=400, budget=4096, cancels=False)
    tight, preemptions, n_tight = run(pages=22, budget=24, cancels=True)
    assert n_free == n_req and n_tight == n_req and set(tight) == set(range(n_req))
    assert preemptions > 0
    for r in range(n_req):
        assert free[r].reason == FINISH_LENGTH and len(free[r].output_tokens) == limits[r]
        if tight[r].reason == FINISH_CANCELLED:
            assert r in cancel_at
            assert tight[r].output_tokens == free[r].output_tokens[:len(tight[r].output_tokens)]
        else:
            assert tight[r].reason == FINISH_LENGTH and tight[r].output_tokens == free[r].output_tokens


@pytest.mark.parametrize("seed", range(8))
def test_a_step_planned_while_the_last_one_runs(seed):
    """The step in two halves: `launched` when it is handed to the device, `resolve` when its sampled values
    arrive, and the next step planned and laid out in between.  With tokens a function of the position, stop
    tokens that do occur, scarce pages (preemption while a value is on its way), cancellations and arrivals at
    random steps, every request ends exactly once with the output and the reason of the run that plans one step
    at a time; no page is lost; a plan that names a sequence which has just ended is dropped."""
    import random
    rng = random.Random(1000 + seed)
    n_req = 14
    prompts = {r: [rng.randrange(1000) for _ in range(rng.randrange(1, 40))] for r in range(n_req)}
    limits = {r: rng.randrange(1, 30) for r in range(n_req)}
    arrive = {r: rng.randrange(0, 25) for r in range(n_req)}
    # a stop token that the request will meet (the token sampled at position p is fake_token(p))
    stops = {r: [fake_token(len(prompts[r]) - 1 + rng.randrange(limits[r]))] if rng.random() < 0.5 else []
             for r in range(n_req)}
    min_tokens = {r: rng.randrange(0, 4) for r in range(n_req)}
    cancel_at = {r: arrive[r] + rng.randrange(0, 12) for r in rng.sample(range(n_req), 3)}

    def sampled_for(plan, batch):
        return [fake_token(int(batch.positions[r])) for r in batch.logits_rows]

    def run(pipelined, pages, budget, cancels):
        sched, cache = make(pages=pages, page_size=4, max_running=4, budget=budget, max_seq_len=60)
        done, step, dropped, ahead = [], 0, 0, None
        while step < 60 or sched.has_work():
            for r in range(n_req):
                if arrive[r] == step:
                    sched.add_request(r, prompts[r], P(limits[r], stop_tokens=stops[r], min_tokens=min_tokens[r]))
                if cancels and cancel_at.get(r) == step:
                    sched.cancel(r)
            if ahead is None:
                plan = sched.prepare_step()
                batch = build_step_batch(cache, plan.entries()) if plan is not None else None
            else:
                plan, batch = ahead
            ahead = None
            if plan is not None:
                assert 0 < plan.num_tokens <= budget and len(plan.contributions) <= 4
                assert all(t >= 0 for t in batch.token_ids.tolist())  # no open place reaches the device
                batch.validate(10 ** 6, [p.num_pages for p in cache.pools], cache.page_size)
                values = sampled_for(plan, batch)
                if not pipelined:
                    sched.commit_step(values)
                else:
                    sched.launched()
                    nxt = sched.prepare_step()  # while the device works
                    nbatch = build_step_batch(cache, nxt.entries()) if nxt is not None else None
                    stale = sched.resolve(values)
                    if nxt is not None and not stale:
                        nbatch.token_ids[:] = sched.plan_token_values(nxt)
                        ahead = (nxt, nbatch)
                    elif nxt is not None:
                        dropped += 1
            done += sched.take_completed()
            cache.check()
            step += 1
            assert step < 5000
        assert all(p.used_pages == 0 for p in cache.pools) and not cache.live_requests()
        assert len(done) == n_req and len({c.rid for c in done}) == n_req
        return {c.rid: c for c in done}, sched.preemptions, dropped

    for pages, budget, cancels in ((400, 4096, False), (22, 24, True), (17, 9, False)):
        one, _, _ = run(False, pages, budget, cancels)
        two, preemptions, dropped = run(True, pages, budget, cancels)
        for r in range(n_req):
            if cancels and r in cancel_at:  # when a cancellation takes hold depends on the step it falls into
                short, long = sorted((one[r].output_tokens, two[r].output_tokens), key=len)
                assert long[:len(short)] == short
            else:
                assert (two[r].output_tokens, two[r].reason) == (one[r].output_tokens, one[r].reason), r
        if pages == 400:
            assert any(c.reason == FINISH_STOP for c in two.values()) and dropped > 0
        else:
            assert preemptions > 0
