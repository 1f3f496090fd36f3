"""The scheduler's decisions (CPU): budget, portions, order, finishing, and what
happens when pages run out. The model is replaced by a rule that makes the next
token a function of the request's tokens so far, and one integration test runs a
toy model through the real step function."""
import copy
import random

import pytest
import torch

import toy_parts  # noqa: F401  (registers the toy architecture)
from pytriton_llama_amd.cache import CacheManager
from pytriton_llama_amd.config import build_model
from pytriton_llama_amd.engine.batch import StepEntry
from pytriton_llama_amd.engine.request import Request, SamplingParams
from pytriton_llama_amd.engine.runner import ModelRunner
from pytriton_llama_amd.engine.scheduler import Scheduler
from pytriton_llama_amd.parts import paged_kv_spec
from pytriton_llama_amd.weights import load_random_weights


def fake_token(req):
    return (sum(req.tokens) * 31 + len(req.tokens)) % 1000


def run(sched, manager, max_steps=10_000, log=None):
    """Drive the scheduler with a stand-in for the step function."""
    steps = 0
    while sched.has_work:
        plan = sched.schedule()
        assert plan.entries
        for e in plan.entries:
            if not manager.is_live(e.request.id):
                manager.admit(e.request.id)
            assert manager.append(e.request.id, e.num_tokens) == e.start
        if log is not None:
            log.append(plan)
        sched.update(plan, {e.request.id: fake_token(e.request) for e in plan.entries if e.samples})
        manager.check()
        steps += 1
        assert steps < max_steps
    return steps


def make(num_pages=64, page=4, seqs=8, budget=32, chunk=None, max_len=None):
    m = CacheManager([paged_kv_spec(1, 16)], page, num_pages, seqs)
    return m, Scheduler(m, seqs, budget, chunk, max_len, eos_token_ids=(999,))


def req(i, n, new=5, **kw):
    return Request(i, list(range(1, n + 1)), SamplingParams(temperature=0, max_new_tokens=new, **kw))


def test_budget_portions_and_decodes_first():
    m, s = make(budget=16, chunk=8)
    reqs = [req(0, 5, 6), req(1, 30, 3), req(2, 11, 4)]
    for r in reqs:
        s.add(r)
    log = []
    run(s, m, log=log)
    for plan in log:
        assert plan.num_tokens <= 16
        kinds = [e.request.remaining == 1 for e in plan.entries]     # before update ... remaining changed
        assert all(e.num_tokens <= 8 for e in plan.entries)
    # first step: request 0 whole (5), then 8 of request 1, then 3 left of the budget for request 2
    first = [(e.request.id, e.start, e.num_tokens, e.samples) for e in log[0].entries]
    assert first == [(0, 0, 5, True), (1, 0, 8, False), (2, 0, 3, False)]
    # second step: request 0 decodes first, prompts share the rest in order of arrival
    second = [(e.request.id, e.num_tokens) for e in log[1].entries]
    assert second == [(0, 1), (1, 8), (2, 7)]
    assert [len(r.output) for r in reqs] == [6, 3, 4]
    assert all(r.status == "finished" and r.finish_reason == "length" for r in reqs)
    assert m.paged[0].pool.num_free == 64 and m.num_free_slots == 8


def test_outputs_do_not_depend_on_the_schedule():
    outs = []
    for budget, chunk, pages in ((64, None, 64), (7, 3, 64), (16, 5, 12)):
        m, s = make(num_pages=pages, budget=budget, chunk=chunk)
        reqs = [req(i, n, 7) for i, n in enumerate([5, 9, 13, 17, 4])]
        for r in reqs:
            s.add(r)
        run(s, m)
        outs.append([r.output for r in reqs])
    assert outs[0] == outs[1] == outs[2]


def test_admission_in_order_of_arrival_and_slots():
    m, s = make(seqs=2, budget=64)
    reqs = [req(i, 6, 2) for i in range(5)]
    for r in reqs:
        s.add(r)
    log = []
    run(s, m, log=log)
    admitted = []
    for plan in log:
        assert len(plan.entries) <= 2
        for e in plan.entries:
            if e.request.id not in admitted:
                admitted.append(e.request.id)
    assert admitted == [0, 1, 2, 3, 4]


def test_a_request_that_does_not_fit_blocks_those_behind_it():
    m, s = make(num_pages=10, page=4, budget=64)      # 40 tokens of cache
    a, b, c = req("a", 30, 2), req("b", 20, 2), req("c", 2, 2)
    for r in (a, b, c):
        s.add(r)
    plan = s.schedule()
    assert [e.request.id for e in plan.entries] == ["a"]     # b does not fit, c must not overtake it


def test_eos_and_max_model_len_finish_a_request():
    m, s = make(max_len=12)
    r = Request("x", [1, 2, 3], SamplingParams(temperature=0, max_new_tokens=9))
    s.add(r)
    plan = s.schedule()
    for e in plan.entries:
        m.admit("x")
        m.append("x", e.num_tokens)
    out = s.update(plan, {"x": 999})
    assert out[0].finished and out[0].finish_reason == "eos" and not m.is_live("x")
    r2 = Request("y", [1, 2, 3], SamplingParams(temperature=0, max_new_tokens=9, ignore_eos=True))
    s.add(r2)
    plan = s.schedule()
    m.admit("y")
    m.append("y", 3)
    assert not s.update(plan, {"y": 999})[0].finished
    with pytest.raises(ValueError, match="max_model_len"):
        s.add(Request("z", [1] * 10, SamplingParams(max_new_tokens=3)))
    with pytest.raises(ValueError, match="empty"):
        s.add(Request("e", [], SamplingParams()))


def _advance(m, plan):
    for e in plan.entries:
        if not m.is_live(e.request.id):
            m.admit(e.request.id)
        assert m.append(e.request.id, e.num_tokens) == e.start


def test_plan_ahead_only_when_every_running_request_decodes_on():
    """The step after a decode step can be planned before its tokens are known: only when all
    running requests decode, nobody waits, no length limit is reached by the token on its way
    and the pages are there; what was planned for a request that then ends is dropped."""
    m, s = make(num_pages=16, page=4, seqs=4, budget=32, max_len=64)
    a, b = req("a", 6, new=4), req("b", 3, new=3)
    s.add(a)
    s.add(b)
    p0 = s.schedule()                                   # both prompts whole
    _advance(m, p0)
    assert s.plan_ahead(p0) is None                     # a prompt step: planned the ordinary way
    s.update(p0, {"a": 5, "b": 6})
    p1 = s.schedule()                                   # both decode
    _advance(m, p1)
    p2 = s.plan_ahead(p1)                               # ... and so they will in the step after
    assert [(e.request.id, e.start, e.num_tokens, e.samples) for e in p2.entries] == \
        [("a", 7, 1, True), ("b", 4, 1, True)]
    _advance(m, p2)                                     # launched before p1's tokens are known
    s.update(p1, {"a": 5, "b": 7})
    assert s.plan_ahead(p2) is None                     # b's token on its way (its third) is its last
    outs = s.update(p2, {"a": 8, "b": 9})
    assert [(o.request, o.finished) for o in outs] == [("a", False), ("b", True)]
    # a request that ends at an end-of-sequence token after the next step was planned
    c = req("c", 2, new=8)
    s.add(c)
    p3 = s.schedule()                                   # a decodes, c's prompt
    _advance(m, p3)
    assert s.plan_ahead(p3) is None
    s.update(p3, {"a": 1, "c": 2})                      # (a's fourth token: a ends by length)
    assert a.status == "finished"
    d = req("d", 3, new=8)
    s.add(d)
    p4 = s.schedule()
    _advance(m, p4)
    s.update(p4, {"c": 3, "d": 4})
    p5 = s.schedule()                                   # c and d decode
    _advance(m, p5)
    p6 = s.plan_ahead(p5)
    assert [e.request.id for e in p6.entries] == ["c", "d"]
    _advance(m, p6)
    s.update(p5, {"c": 999, "d": 5})                    # c ends here
    assert c.status == "finished" and not m.is_live("c")
    assert s.plan_ahead(p6) is None                     # p6 no longer covers the running requests
    outs = s.update(p6, {"c": 123, "d": 6})             # what p6 computed for c is dropped
    assert [(o.request, o.token) for o in outs] == [("d", 6)]
    assert c.output == [2, 3, 999] and d.output == [4, 5, 6]
    m.check()
    # somebody waits: no planning ahead
    p7 = s.schedule()
    _advance(m, p7)
    s.add(req("e", 2, new=2))
    assert s.plan_ahead(p7) is None
    # no page for the token after next: no planning ahead
    m2, s2 = make(num_pages=4, page=4, seqs=2, budget=32)
    r, other = req("r", 7, new=6), req("o", 5, new=2)
    s2.add(r)
    s2.add(other)
    q0 = s2.schedule()                                  # r: two pages, o: two pages: none is left
    _advance(m2, q0)
    s2.update(q0, {"r": 1, "o": 1})
    q1 = s2.schedule()                                  # r at position 7, the last of its second page
    _advance(m2, q1)
    assert m2.paged[0].pool.num_free == 0
    assert s2.plan_ahead(q1) is None                    # position 8 would need a page that is not there


def test_planning_ahead_gives_the_same_outputs():
    """Driving the scheduler one step ahead wherever it allows gives every request the tokens
    it gets step by step."""
    def drive(ahead):
        m, s = make(num_pages=40, page=4, seqs=4, budget=24, chunk=8, max_len=80)
        reqs = [req(i, n, new=k) for i, (n, k) in enumerate([(5, 9), (17, 4), (9, 12), (3, 7)])]
        for r in reqs[:3]:
            s.add(r)
        pending, steps, late = None, 0, reqs[3]
        while s.has_work or pending is not None:
            if pending is None:
                pending = s.schedule()
                _advance(m, pending)
            cur, nxt = pending, None
            if ahead:
                nxt = s.plan_ahead(cur)
                if nxt is not None:
                    _advance(m, nxt)
            toks = {e.request.id: (e.start * 7 + 3) % 50 for e in cur.entries if e.samples}
            s.update(cur, toks)
            m.check()
            pending = nxt
            steps += 1
            if steps == 6:
                s.add(late)
            assert steps < 500
        assert m.paged[0].pool.num_free == 40
        return [r.output for r in reqs]
    assert drive(True) == drive(False)


def test_a_request_that_can_never_fit_is_refused():
    m, s = make(num_pages=4, page=4)
    with pytest.raises(ValueError, match="never fit"):
        s.add(req("big", 10, 8))
    s.add(req("ok", 10, 6))


def test_pages_run_out_the_latest_request_is_preempted_and_recomputed():
    m, s = make(num_pages=9, page=4, budget=64)      # 36 tokens
    a, b = req("a", 14, 12), req("b", 14, 12)         # each needs 26 in the end: both cannot finish together
    s.add(a)
    s.add(b)
    log = []
    run(s, m, log=log)
    assert s.num_preemptions >= 1 and b.num_preemptions >= 1 and a.num_preemptions == 0
    pre = [p for p in log if p.preempted]
    assert all(v is b for p in pre for v in p.preempted)
    # the step that preempts b still runs a
    assert all(any(e.request is a for e in p.entries) for p in pre)
    # b comes back with its generated tokens as part of what is recomputed
    i = log.index(pre[0])
    back = next(p for p in log[i + 1:] if any(e.request is b for e in p.entries))
    e = next(e for e in back.entries if e.request is b)
    assert e.start == 0 and e.num_tokens > 14
    # and the outputs are those of an undisturbed run
    m2, s2 = make(num_pages=64, page=4, budget=64)
    a2, b2 = req("a", 14, 12), req("b", 14, 12)
    s2.add(a2)
    s2.add(b2)
    run(s2, m2)
    assert (a.output, b.output) == (a2.output, b2.output) and s2.num_preemptions == 0


@pytest.mark.parametrize("seed", range(6))
def test_random_loads_finish_within_budget(seed):
    rng = random.Random(seed)
    page = rng.choice([1, 4, 16])
    budget = rng.randint(4, 40)
    m, s = make(num_pages=rng.randint(60 // page + 2, 200 // page + 2), page=page,
                seqs=rng.randint(1, 6), budget=budget, chunk=rng.choice([None, 2, 5, 16]))
    reqs = [req(i, rng.randint(1, 40), rng.randint(1, 12)) for i in range(12)]
    for r in reqs:
        s.add(r)
    log = []
    run(s, m, log=log)
    assert all(p.num_tokens <= budget for p in log)
    assert all(r.status == "finished" and len(r.output) == r.params.max_new_tokens for r in reqs)
    m2, s2 = make(num_pages=4000, page=1, seqs=12, budget=4000)
    ref = [req(i, len(r.prompt), r.params.max_new_tokens) for i, r in enumerate(reqs)]
    for r in ref:
        s2.add(r)
    run(s2, m2)
    assert [r.output for r in reqs] == [r.output for r in ref]
    assert m.paged[0].pool.num_free == m.paged[0].pool.num_pages


TOY = {"architectures": ["ToyStateLM"], "vocab_size": 50, "hidden_size": 12, "inner": 20,
       "layers": ["state", "state"], "order": [0, 1, 0], "decay": 0.8, "toy_norm": True,
       "toy_ffn": True}


def test_toy_model_with_state_through_the_real_step_function():
    """A mixer with state of its own (no pages), a layer named twice in the run
    order: registered from the test, built by the registry, stepped by the
    runner in any cutting, and scheduled with preemption."""
    model = build_model(copy.deepcopy(TOY))
    load_random_weights(model, 5, torch.float32, "cpu")
    assert len(model.cache_layers) == 3 and len(model.blocks) == 2
    runner = ModelRunner(model, page_size=4, num_pages=4, max_num_seqs=3)
    assert len(runner.manager.states) == 1 and runner.manager.states[0].layers == [0, 1, 2]
    seq = [3, 14, 15, 9, 2, 6, 5, 35, 8, 9, 7, 9]
    want = toy_parts.toy_plain_forward(model, seq)
    # whole
    got = runner.step([StepEntry("w", seq, list(range(len(seq))))])
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    runner.end("w")
    # cut, beside another request that lives in another slot
    other = [1, 2, 3, 4, 5, 6]
    rows = []
    rows.append(runner.step([StepEntry("c", seq[:5], [0, 1, 2, 3, 4]), StepEntry("o", other[:2], [])]))
    rows.append(runner.step([StepEntry("o", other[2:], []), StepEntry("c", seq[5:6], [0])])[-1:])
    rows.append(runner.step([StepEntry("c", seq[6:], list(range(6)))]))
    torch.testing.assert_close(torch.cat(rows), want, atol=1e-5, rtol=1e-5)
    runner.end("c")
    runner.end("o")
    # a new request in a used slot starts from zero state
    again = runner.step([StepEntry("n", seq, [len(seq) - 1])])
    torch.testing.assert_close(again[0], want[-1], atol=1e-5, rtol=1e-5)
