"""The scheduler's decisions, with a fake model step (no GPU)."""
import random

import pytest

from pico_vllm_amd.cache.manager import CacheManager
from pico_vllm_amd.engine.request import Request, RequestStatus
from pico_vllm_amd.engine.scheduler import Scheduler
from pico_vllm_amd.parts.attention import kv_page_tensors
from pico_vllm_amd.parts.spec import CacheSpec
from pico_vllm_amd.sampling.params import SamplingParams
from pico_vllm_amd.sampling.sampler import uniform

SPEC = {0: CacheSpec("paged_kv", page_tensors=kv_page_tensors(1, 16))}


def make(num_pages=64, page=16, max_seqs=4, budget=32, max_len=512):
    m = CacheManager(SPEC, page, num_pages, max_seqs)
    return m, Scheduler(m, max_seqs, budget, max_len)


def req(i, n_prompt, n_new):
    return Request(i, list(range(1, n_prompt + 1)), SamplingParams(max_new_tokens=n_new))


def drive(s: Scheduler, requests, max_steps=10000, log=None):
    """Run to completion with a fake step: the 'sampled' token is a function of what was run."""
    order = []
    for _ in range(max_steps):
        if not s.has_unfinished():
            return order
        plan = s.schedule()
        assert plan.seqs, "nothing scheduled although requests are unfinished"
        assert plan.num_tokens <= s.max_num_batched_tokens
        assert len(s.running) <= s.max_num_seqs
        if log is not None:
            log.append([(x.request.request_id, x.request.num_computed, x.num_tokens) for x in plan.seqs])
        for x in plan.seqs:
            samples = x.samples
            s.on_step_done(x)
            if samples:
                r = x.request
                r.generated_ids.append((sum(r.all_ids) * 31 + len(r.all_ids)) % 1000)
                if r.is_max_len_finished():
                    s.finish(r, "length")
                    order.append(r.request_id)
        s.manager.check()
    raise AssertionError("did not finish")


def test_a_prompt_portion_is_capped_beside_the_budget():
    # prefill_chunk: the longest portion of ONE prompt in a step; the budget is what all sequences of a step share
    m = CacheManager(SPEC, 16, 64, 4)
    s = Scheduler(m, 4, 32, 512, prefill_chunk=12)
    for i, n in enumerate([30, 10, 29]):
        s.add_request(req(i, n, 2))
    log = []
    drive(s, None, log=log)
    assert log[0] == [(0, 0, 12), (1, 0, 10), (2, 0, 10)]                  # 12 of request 0, then the budget's rest
    assert log[1] == [(0, 12, 12), (1, 10, 1), (2, 10, 12)] or log[1] == [(1, 10, 1), (0, 12, 12), (2, 10, 12)]
    assert all(n <= 12 for step in log for _, _, n in step)
    assert all(sum(n for _, _, n in step) <= 32 for step in log)
    # the cap never exceeds the budget, and nonsense is refused
    assert Scheduler(m, 4, 32, 512, prefill_chunk=100).prefill_chunk == 32 and Scheduler(m, 4, 32, 512).prefill_chunk == 32
    with pytest.raises(ValueError, match="prefill_chunk"):
        Scheduler(m, 4, 32, 512, prefill_chunk=0)


def test_fcfs_admission_and_token_budget_cut_prompts_into_portions():
    m, s = make(budget=32, max_seqs=4)
    for i, n in enumerate([50, 10, 70]):
        s.add_request(req(i, n, 3))
    log = []
    drive(s, None, log=log)
    # step 0: request 0 gets the whole budget; request 1 is not admitted before request 0's turn is served
    assert log[0] == [(0, 0, 32)]
    assert log[1] == [(0, 32, 18), (1, 0, 10), (2, 0, 4)]
    # decode tokens come first afterwards, then the prompt portion of request 2
    assert log[2][:2] == [(0, 50, 1), (1, 10, 1)] and log[2][2] == (2, 4, 30)


def test_finishing_frees_pages_in_the_same_step_and_first_token_counts():
    m, s = make()
    s.add_request(req(0, 5, 1))
    plan = s.schedule()
    assert plan.seqs[0].samples and plan.seqs[0].num_tokens == 5
    s.on_step_done(plan.seqs[0])
    plan.seqs[0].request.generated_ids.append(7)
    assert plan.seqs[0].request.is_max_len_finished()       # max_new_tokens = 1: done after the prefill step
    s.finish(plan.seqs[0].request, "length")
    assert not s.has_unfinished() and m.groups[0].pool.num_free == 64 and m.slots.num_free == 4
    assert plan.seqs[0].request.status is RequestStatus.FINISHED


def test_request_that_can_never_fit_is_refused_at_once():
    m, s = make(num_pages=4, page=16)
    with pytest.raises(ValueError, match="never finish"):
        s.add_request(req(0, 60, 10))
    with pytest.raises(ValueError, match="max_seq_len"):
        make(max_len=32)[1].add_request(req(0, 30, 10))
    s.add_request(req(1, 60, 4))                              # exactly 4 pages


def test_pages_running_out_preempts_the_last_admitted_which_recomputes():
    m, s = make(num_pages=6, page=16, max_seqs=3, budget=64)
    a, b = req(0, 30, 40), req(1, 30, 40)                      # each grows to 70 tokens = 5 pages; pool has 6
    s.add_request(a); s.add_request(b)
    log = []
    done = drive(s, None, log=log)
    assert done == [0, 1]                                      # the older request is never the victim
    assert b.num_preemptions >= 1 and a.num_preemptions == 0 and s.num_preemptions == b.num_preemptions
    # after its preemption, b ran its prompt AND its generated tokens again from position 0
    restart = [e for step in log for e in step if e[0] == 1 and e[1] == 0]
    assert len(restart) == 1 + b.num_preemptions and restart[-1][2] > 30
    assert len(a.generated_ids) == 40 and len(b.generated_ids) == 40
    # the same tokens as with plenty of pages: the fake token depends only on the request's own history
    m2, s2 = make(num_pages=64, page=16, max_seqs=3, budget=64)
    a2, b2 = req(0, 30, 40), req(1, 30, 40)
    s2.add_request(a2); s2.add_request(b2)
    drive(s2, None)
    assert a2.generated_ids == a.generated_ids and b2.generated_ids == b.generated_ids
    assert m.groups[0].pool.reuse_count > 0


def test_no_admission_without_pages_or_slots():
    m, s = make(num_pages=4, page=16, max_seqs=2, budget=64)
    s.add_request(req(0, 40, 2)); s.add_request(req(1, 40, 2)); s.add_request(req(2, 5, 2))
    plan = s.schedule()
    # request 0 takes 3 of 4 pages; request 1 needs 3: not admitted, and request 2 does not jump the queue
    assert [x.request.request_id for x in plan.seqs] == [0]
    assert [r.request_id for r in s.waiting] == [1, 2]


@pytest.mark.parametrize("seed", range(5))
def test_every_request_finishes_under_random_load_and_a_tiny_pool(seed):
    rng = random.Random(seed)
    m, s = make(num_pages=12, page=8, max_seqs=4, budget=24, max_len=96)
    reqs = [req(i, rng.randint(1, 40), rng.randint(1, 30)) for i in range(12)]
    for r in reqs:
        s.add_request(r)
    done = drive(s, None)
    assert sorted(done) == list(range(12))
    assert all(len(r.generated_ids) == r.params.max_new_tokens for r in reqs)
    assert m.groups[0].pool.num_free == 12 and m.slots.num_free == 4


def test_uniform_numbers_are_a_pure_function_of_seed_and_index():
    a = [uniform(5, i) for i in range(1000)]
    assert a == [uniform(5, i) for i in range(1000)] and a != [uniform(6, i) for i in range(1000)]
    assert all(0.0 <= x < 1.0 for x in a) and 0.45 < sum(a) / 1000 < 0.55


def test_a_token_that_the_host_has_not_read_yet_counts_as_a_token():
    # the decode pipeline starts a step before the tokens of the step before it are known: the request
    # then carries them as pending; the scheduler plans with them, the values arrive later
    m, s = make()
    r = req(0, 5, 4)
    s.add_request(r)
    plan = s.schedule()
    assert plan.seqs[0].num_tokens == 5 and plan.seqs[0].samples
    s.on_step_done(plan.seqs[0])
    r.num_pending += 1                                  # sampled on the device, not read
    assert r.total_len == 6 and r.num_uncomputed == 1 and r.num_generated == 1 and r.all_ids == [1, 2, 3, 4, 5]
    plan = s.schedule()                                 # the next decode step can be planned already
    assert [(x.request.request_id, x.num_tokens, x.samples) for x in plan.seqs] == [(0, 1, True)]
    s.on_step_done(plan.seqs[0])
    r.num_pending += 1
    assert r.num_computed == 6 and r.total_len == 7
    r.num_pending -= 1
    r.generated_ids.append(11)                          # the first value arrives
    assert r.total_len == 7 and r.all_ids[-1] == 11 and not r.is_max_len_finished()
    m.check()


def test_a_preempted_request_can_finish_while_it_waits():
    # its last token was still on the device when it was preempted and turns out to end it
    m, s = make(num_pages=4, page=16, max_seqs=2, budget=64)
    a, b = req(0, 30, 30), req(1, 30, 30)
    s.add_request(a)
    s.add_request(b)
    for x in s.schedule().seqs:
        s.on_step_done(x)
        x.request.num_pending += 1
    for _ in range(40):                                 # decode until the pool runs dry and b is preempted
        plan = s.schedule()
        if plan.preempted:
            break
        for x in plan.seqs:
            s.on_step_done(x)
            x.request.num_pending -= 1
            x.request.generated_ids.append(3)
            x.request.num_pending += 1
    assert plan.preempted == [b] and b.status is RequestStatus.WAITING and b.num_pending == 1
    s.finish(b, "eos")
    assert b.status is RequestStatus.FINISHED and list(s.waiting) == [] and s.running == [a]
    m.check()



def test_a_windowed_group_is_sized_by_its_window_not_by_the_length():
    # layers that read only the last 40 keys hold 40 + a step's tokens, whatever the length of the request: a pool
    # of 8 pages (128 tokens) serves a request of 400 tokens, which a group without a window would refuse
    win = {0: CacheSpec("paged_kv", window=40, page_tensors=kv_page_tensors(1, 16))}
    m = CacheManager(win, 16, 8, 2)
    s = Scheduler(m, 2, 32, 512)
    s.add_request(req(0, 300, 100))
    order = drive(s, None)
    assert order == [0] and m.groups[0].pool.num_free == 8 and m.groups[0].pool.peak_used <= 6
    full, s2 = make(num_pages=8, budget=32, max_seqs=2)
    with pytest.raises(ValueError, match="could never finish"):
        s2.add_request(req(1, 300, 100))


def test_no_admission_without_a_state_slot_and_what_the_scheduler_refuses():
    m = CacheManager(SPEC, 16, 64, 1)                       # one slot for per-request state, though two may run
    s = Scheduler(m, 2, 64, 512)
    s.add_request(req(0, 5, 3)); s.add_request(req(1, 5, 3))
    assert [x.request.request_id for x in s.schedule().seqs] == [0] and [r.request_id for r in s.waiting] == [1]
    assert drive(s, None) == [0, 1]                         # the second one runs when the first has given its slot back
    with pytest.raises(ValueError, match="starve"):
        Scheduler(m, 8, 4, 512)
    with pytest.raises(ValueError, match="at least one prompt token"):
        s.add_request(Request(2, [], SamplingParams(max_new_tokens=1)))
    with pytest.raises(ValueError, match="exceeds max_seq_len"):
        s.add_request(req(3, 510, 3))


@pytest.mark.parametrize("field,value", [("max_new_tokens", 0), ("max_new_tokens", 2.5), ("max_new_tokens", True),
                                         ("temperature", -0.1), ("temperature", float("nan")), ("temperature", float("inf")),
                                         ("top_p", 0.0), ("top_p", float("nan")), ("top_p", -1.0),
                                         ("stop_token_ids", [3, "4"]), ("stop_token_ids", [1.0])])
def test_sampling_options_that_make_no_sense_are_refused(field, value):
    SamplingParams().validate()
    SamplingParams(max_new_tokens=1, temperature=0.0, top_p=1.0).validate()
    SamplingParams(temperature=3, top_p=5, stop_token_ids=[0, 7]).validate()       # top_p >= 1: no nucleus filter
    with pytest.raises(ValueError, match=field):
        SamplingParams(**{field: value}).validate()
