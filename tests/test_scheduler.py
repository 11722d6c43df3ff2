"""The scheduler's decisions on the host: admission, portions under a token budget, decoding
first, finishing, and pre-emption when pages run out."""
import pytest

from swifttransformer_amd.cache import CacheManager
from swifttransformer_amd.engine.scheduler import FINISHED, RUNNING, WAITING, Request, Scheduler
from swifttransformer_amd.parts import CacheNeed
from swifttransformer_amd.sampling import SamplingParams

FULL = CacheNeed("paged_kv", num_kv_heads=2, head_dim=16)


def make(num_pages=64, page_size=4, max_seqs=4, budget=32, chunk=16, max_positions=128, eos=2):
    m = CacheManager({0: FULL, 1: FULL}, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs,
                     max_pages_per_seq=-(-max_positions // page_size))
    s = Scheduler(m, max_batched_tokens=budget, prefill_chunk=chunk, max_positions=max_positions,
                  eos_token_id=eos)
    return m, s


def req(i, n, **kw):
    return Request(i, list(range(10, 10 + n)), SamplingParams(**kw))


def run_step(s, token=7):
    sch = s.schedule()
    fin = s.update(sch, {x.request.req_id: token for x in sch if x.sample})
    return sch, fin


def test_portions_budget_and_decode_first():
    m, s = make(budget=20, chunk=16)
    s.add(req("a", 30, max_new_tokens=3))
    s.add(req("b", 5, max_new_tokens=3))
    sch, _ = run_step(s)
    # a gets a 16-token portion, b its first 4 tokens (budget 20)
    assert [(x.request.req_id, x.start, len(x.tokens), x.sample) for x in sch] == \
        [("a", 0, 16, False), ("b", 0, 4, False)]
    sch, _ = run_step(s)
    # requests with a single token to run come first, then the rest of a's prompt
    assert [(x.request.req_id, x.start, len(x.tokens), x.sample) for x in sch] == \
        [("b", 4, 1, True), ("a", 16, 14, True)]
    sch, _ = run_step(s)
    # both decode now: one token each, positions follow on
    assert [(x.request.req_id, x.start, x.tokens, x.sample) for x in sch] == \
        [("a", 30, [7], True), ("b", 5, [7], True)]
    m.check_invariants()
    # a new arrival is admitted beside the decoding ones, decode tokens first in the batch
    s.add(req("c", 40, max_new_tokens=2))
    sch, fin = run_step(s)
    assert [x.request.req_id for x in sch] == ["a", "b", "c"]
    assert [len(x.tokens) for x in sch] == [1, 1, 16]
    assert {r.req_id for r in fin} == {"a", "b"} and all(r.finish_reason == "length" for r in fin)
    assert all(r.status == FINISHED for r in fin)
    m.check_invariants()


def test_finish_on_eos_and_ignore_eos():
    m, s = make()
    s.add(req("a", 3, max_new_tokens=10))
    s.add(req("b", 3, max_new_tokens=2, ignore_eos=True))
    _, fin = run_step(s, token=2)
    assert [r.req_id for r in fin] == ["a"] and fin[0].finish_reason == "eos" and fin[0].output == [2]
    _, fin = run_step(s, token=2)
    assert [r.req_id for r in fin] == ["b"] and fin[0].finish_reason == "length"
    assert not s.has_work() and m.num_free_pages(0) == 64 and m.num_free_slots == 4


def test_positions_run_out():
    m, s = make(max_positions=8, budget=64, chunk=64)
    s.add(req("a", 6, max_new_tokens=50, ignore_eos=True))
    outs = []
    while s.has_work():
        _, fin = run_step(s, token=5)
        outs += fin
    # tokens at positions 6 and 7 can be run; the one after has no position left
    assert outs[0].finish_reason == "positions" and len(outs[0].output) == 3
    with pytest.raises(ValueError, match="exceeds the model"):
        s.add(req("b", 9))


def test_slots_limit_admission():
    m, s = make(max_seqs=2)
    for i in range(3):
        s.add(req(i, 4, max_new_tokens=2, ignore_eos=True))
    sch, _ = run_step(s)
    assert [x.request.req_id for x in sch] == [0, 1]
    sch, fin = run_step(s)
    assert len(fin) == 2
    sch, _ = run_step(s)
    assert [x.request.req_id for x in sch] == [2]


def test_preemption_when_pages_run_out_and_same_output():
    """Two requests whose growth exhausts the pool: the later one is pre-empted, recomputed
    from prompt+output, and every request still gets its full output."""
    m, s = make(num_pages=9, page_size=4, budget=64, chunk=64)
    s.add(req("a", 14, max_new_tokens=12, ignore_eos=True))   # needs up to 7 pages
    s.add(req("b", 9, max_new_tokens=10, ignore_eos=True))    # needs up to 5 pages
    done = {}
    steps = 0
    while s.has_work():
        sch = s.schedule()
        assert sch, "no progress"
        # the "model": next token = 100 + position of the sampled row (depends on nothing else)
        fin = s.update(sch, {x.request.req_id: 100 + x.start + len(x.tokens) - 1 for x in sch if x.sample})
        for r in fin:
            done[r.req_id] = r
        m.check_invariants()
        steps += 1
        assert steps < 200
    assert s.num_preemptions >= 1 and done["b"].preemptions >= 1 and done["a"].preemptions == 0
    assert done["a"].output == [100 + 13 + i for i in range(12)]
    assert done["b"].output == [100 + 8 + i for i in range(10)]
    assert m.num_free_pages(0) == 9


def test_request_that_can_never_fit_is_refused():
    m, s = make(num_pages=4, page_size=4)
    with pytest.raises(ValueError, match="may need"):
        s.add(req("a", 10, max_new_tokens=20))
    s.add(req("b", 10, max_new_tokens=6))
    assert s.has_work()


def test_waiting_request_waits_for_pages_not_forever():
    m, s = make(num_pages=8, page_size=4, budget=64, chunk=64)
    s.add(req("a", 20, max_new_tokens=4, ignore_eos=True))     # 6 pages
    s.add(req("b", 20, max_new_tokens=4, ignore_eos=True))     # cannot start beside a
    sch, _ = run_step(s)
    assert [x.request.req_id for x in sch] == ["a"] and s.waiting[0].req_id == "b"
    order = []
    while s.has_work():
        sch, fin = run_step(s)
        order += [r.req_id for r in fin]
    assert order == ["a", "b"]
