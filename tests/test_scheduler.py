"""The scheduler's decisions, on the host, with a stand-in for the model (the next token
is a function of the request's tokens so far)."""
import pytest

from nano_vllm_amd.cache import CacheGroup, CacheManager
from nano_vllm_amd.engine.scheduler import Scheduler
from nano_vllm_amd.engine.sequence import Sequence, SequenceStatus
from nano_vllm_amd.sampling.params import SamplingParams


def _sched(pages=16, page=4, max_seqs=8, budget=16, max_len=64, eos=(), policy="prefill_first", prefix=True):
    cache = CacheManager([CacheGroup(None, (0,))], page, pages, enable_prefix_caching=prefix)
    return Scheduler(cache, max_seqs, budget, max_len, eos, policy)


def _seq(n, base=0, **kw):
    return Sequence([base + i for i in range(n)], SamplingParams(**({"temperature": 0.0, "max_tokens": 4} | kw)))


def _next_token(seq):
    return (sum(seq.token_ids) * 31 + len(seq)) % 97 + 100


def _run(s, check_each=True):
    """Drives the scheduler to the end; returns the batches it chose as [(seq_id, start, n)]."""
    log = []
    for _ in range(10000):
        if s.is_finished():
            return log
        seqs, is_prefill = s.schedule()
        log.append((is_prefill, [(q.seq_id, q.num_cached_tokens, q.num_scheduled_tokens) for q in seqs]))
        s.postprocess(seqs, [_next_token(q) for q in seqs])
        if check_each:
            s.cache.check()
    raise AssertionError("the scheduler does not end")


def test_whole_prompts_share_a_step_and_then_decode():
    s = _sched()
    a, b = _seq(5), _seq(7, 50)
    s.add(a); s.add(b)
    seqs, pre = s.schedule()
    assert pre and [(q.num_cached_tokens, q.num_scheduled_tokens) for q in seqs] == [(0, 5), (0, 7)]
    s.postprocess(seqs, [1, 2])
    assert a.status == SequenceStatus.RUNNING and a.num_tokens == 6 and a.num_cached_tokens == 5
    seqs, pre = s.schedule()
    assert not pre and [q.num_scheduled_tokens for q in seqs] == [1, 1]


def test_only_the_first_prompt_of_a_step_is_cut():
    s = _sched(budget=8)                                     # scheduler.py:42-43
    a, b = _seq(5), _seq(7, 50)
    s.add(a); s.add(b)
    seqs, _ = s.schedule()
    assert [(q.seq_id, q.num_scheduled_tokens) for q in seqs] == [(a.seq_id, 5)]   # b does not fit and is not first
    s.postprocess(seqs, [1])
    seqs, pre = s.schedule()                                 # prefill goes before decode
    assert pre and [(q.seq_id, q.num_scheduled_tokens) for q in seqs] == [(b.seq_id, 7)]
    s = _sched(budget=8)
    c = _seq(19)
    s.add(c)
    cuts = []
    while c.status == SequenceStatus.WAITING:
        seqs, _ = s.schedule()
        cuts.append((seqs[0].num_cached_tokens, seqs[0].num_scheduled_tokens))
        s.postprocess(seqs, [1])
    assert cuts == [(0, 8), (8, 8), (16, 3)]
    assert c.num_tokens == 20                                # a token only after the last portion


def test_token_budget_and_request_limit_hold():
    s = _sched(pages=64, budget=10, max_seqs=2)
    for i in range(5):
        s.add(_seq(4, 10 * i))
    for is_prefill, batch in _run(s):
        assert len(batch) <= 2 and sum(n for _, _, n in batch) <= 10


def test_finishing_frees_pages_and_respects_eos_and_max_tokens():
    s = _sched(eos=(7,))
    a = _seq(5, max_tokens=3)
    b = _seq(5, 50, max_tokens=9)
    c = _seq(5, 20, max_tokens=9, ignore_eos=True)
    for q in (a, b, c):
        s.add(q)
    seqs, _ = s.schedule()
    s.postprocess(seqs, [1, 7, 7])                           # b meets eos, c ignores it
    assert b.is_finished and b.finish_reason == "eos" and b.completion_token_ids == [7]
    assert not c.is_finished
    while not s.is_finished():
        seqs, _ = s.schedule()
        s.postprocess(seqs, [3] * len(seqs))
    assert a.finish_reason == "max_tokens" and a.num_completion_tokens == 3
    assert c.num_completion_tokens == 9
    assert s.cache.pools[0].num_free == 16
    s.cache.check()


def test_max_model_len_ends_a_request():
    s = _sched(max_len=8)
    a = _seq(5, max_tokens=50)
    s.add(a)
    _run(s)
    assert a.finish_reason == "length" and a.num_tokens == 8
    with pytest.raises(ValueError, match="max_model_len"):
        s.add(_seq(8))


def test_waiting_request_stays_at_the_head_until_pages_are_free():
    s = _sched(pages=4, page=4)
    a, b = _seq(9, max_tokens=2), _seq(9, 50, max_tokens=2)  # 3 pages each
    s.add(a); s.add(b)
    seqs, _ = s.schedule()
    assert [q.seq_id for q in seqs] == [a.seq_id]            # b's pages are not free (scheduler.py:37-38)
    s.postprocess(seqs, [1])
    seqs, pre = s.schedule()
    assert not pre and [q.seq_id for q in seqs] == [a.seq_id]
    s.postprocess(seqs, [1])                                 # a ends and frees its pages
    seqs, pre = s.schedule()
    assert pre and [q.seq_id for q in seqs] == [b.seq_id]


def test_the_newest_running_request_is_preempted_and_computed_again():
    s = _sched(pages=4, page=4, prefix=False)
    a, b = _seq(4, max_tokens=8), _seq(7, 50, max_tokens=8)
    s.add(a); s.add(b)
    seqs, _ = s.schedule()
    s.postprocess(seqs, [_next_token(q) for q in seqs])      # a holds 1 page (4 tokens), b 2 pages (7)
    seqs, _ = s.schedule()                                   # a needs a 2nd page, b writes into its 2nd
    assert len(seqs) == 2
    s.postprocess(seqs, [_next_token(q) for q in seqs])      # a: 6 tokens, b: 9 tokens
    seqs, _ = s.schedule()                                   # b needs a 3rd page: the pool (4) is full
    # the newest running request (b) is taken from (scheduler.py:60-65,75-79)
    assert [q.seq_id for q in seqs] == [a.seq_id] and s.num_preemptions == 1
    assert b.status == SequenceStatus.WAITING and b.num_cached_tokens == 0 and s.waiting[0] is b
    assert b.num_tokens == 9                                 # its generated tokens are kept
    s.cache.check()
    s.postprocess(seqs, [_next_token(q) for q in seqs])
    _run(s)
    # the same continuation as without a shortage
    s2 = _sched(pages=64, page=4, prefix=False)
    a2, b2 = _seq(4, max_tokens=8), _seq(7, 50, max_tokens=8)
    s2.add(a2); s2.add(b2)
    _run(s2)
    assert a.token_ids == a2.token_ids and b.token_ids == b2.token_ids and s2.num_preemptions == 0


def test_a_request_alone_that_cannot_grow_is_finished_not_asserted():
    s = _sched(pages=2, page=4, max_len=64)
    a = _seq(6, max_tokens=30)
    s.add(a)
    _run(s)
    assert a.finish_reason == "cache_full" and a.num_tokens == 9     # 8 positions cached + the token that found no page
    assert s.cache.pools[0].num_free == 2
    with pytest.raises(ValueError, match="pages"):
        s.add(_seq(9))                                       # can never fit 2 pages


def test_prefix_hits_shorten_the_prompt_portion():
    s = _sched(pages=16, page=4)
    a = _seq(10, max_tokens=1)
    s.add(a)
    _run(s)
    b = Sequence(list(range(10)) + [77], SamplingParams(temperature=0.0, max_tokens=1))
    s.add(b)
    seqs, _ = s.schedule()
    assert (seqs[0].num_cached_tokens, seqs[0].num_scheduled_tokens) == (8, 3)      # two pages found


@pytest.mark.parametrize("policy", ["prefill_first", "mixed"])
def test_policies_end_with_the_same_tokens(policy):
    def run(policy, pages):
        s = _sched(pages=pages, page=4, budget=6, max_seqs=3, policy=policy, prefix=False)
        seqs = [_seq(n, 10 * n, max_tokens=6) for n in (3, 9, 14, 5, 11)]
        for q in seqs:
            s.add(q)
        log = _run(s)
        return [q.token_ids for q in seqs], log, s
    want, _, _ = run("prefill_first", 64)
    got, log, s = run(policy, 9)
    assert got == want
    assert s.cache.pools[0].num_free == 9
    if policy == "mixed":
        assert any(len({n for _, _, n in b}) > 1 and any(n == 1 for _, _, n in b) for _, b in log), \
            "no step mixed a prompt portion with decoded tokens"


def test_mixed_policy_takes_pages_from_a_prompt_that_is_still_being_cut():
    """Under "mixed" the request admitted last may hold pages while it is still at the head of
    the waiting queue (its prompt goes in portions).  A running request that needs a page takes
    them from it, the newest, instead of ending with "cache_full"; it is computed again later."""
    def run(policy, pages):
        s = _sched(pages=pages, page=4, budget=3, policy=policy, prefix=False)
        a, b = _seq(3, max_tokens=12), _seq(16, 50, max_tokens=3)
        s.add(a); s.add(b)
        log = _run(s)
        return a, b, s, log
    a, b, s, log = run("mixed", 6)           # a grows to 4 pages while b holds 4 for its 16-token prompt
    assert s.num_preemptions >= 1
    assert a.finish_reason == "max_tokens" and a.num_completion_tokens == 12
    assert b.finish_reason == "max_tokens" and b.num_completion_tokens == 3
    assert s.cache.pools[0].num_free == 6
    # b was taken from while part of its prompt was in the cache, and kept its place in the queue
    assert any(sid == b.seq_id and start > 0 for _, batch in log for sid, start, n in batch)
    a2, b2, s2, _ = run("prefill_first", 64)
    assert a.token_ids == a2.token_ids and b.token_ids == b2.token_ids and s2.num_preemptions == 0


def test_admission_is_sized_group_by_group():
    """A window group holds the pages of one step's tokens and of the window before them, never
    the whole prompt: a prompt longer than that group's pool is admitted and runs to the end, and
    one that the all-keys group cannot hold is refused with the group named."""
    groups = [CacheGroup(None, (0,)), CacheGroup(6, (1,))]
    cache = CacheManager(groups, 4, [16, 4], enable_prefix_caching=False)
    assert cache.peak_pages(41, 8) == [11, 4]         # 6 - 1 + 8 positions at any offset: 4 pages of 4
    assert cache.peak_pages(3, 8) == [1, 1]
    s = Scheduler(cache, 4, 8, 64, (), "prefill_first")
    q = _seq(40)
    s.add(q)                                          # 11 pages of all keys; the window group has 4 in all
    _run(s)
    assert q.is_finished and q.num_completion_tokens == 4
    assert cache.pools[0].num_free == 16 and cache.pools[1].num_free == 4
    small = Scheduler(CacheManager(groups, 4, [16, 3], enable_prefix_caching=False), 4, 8, 64, (), "prefill_first")
    with pytest.raises(ValueError, match="cache group 1"):
        small.add(_seq(40))
    with pytest.raises(ValueError, match="cache group 0"):
        Scheduler(CacheManager(groups, 4, [8, 4], enable_prefix_caching=False), 4, 8, 64, (), "prefill_first").add(_seq(40))


def test_a_short_prompt_that_decodes_across_the_window_is_sized_for_the_window():
    """The window group's need while decoding (a whole window, at any offset) is checked when the
    request is added, not found out later as cache_full: a prompt of 3 tokens fits one page, but
    its 30 decoded tokens need the pages of a window of 10."""
    groups = [CacheGroup(None, (0,)), CacheGroup(10, (1,))]
    # 10 positions at any offset touch 4 pages of 4 (the worst: a window that starts on a page's last slot)
    assert CacheManager(groups, 4, [16, 4], enable_prefix_caching=False).peak_pages(33, 1) == [9, 4]
    with pytest.raises(ValueError, match="cache group 1"):
        Scheduler(CacheManager(groups, 4, [16, 3], enable_prefix_caching=False), 4, 8, 64, (), "prefill_first").add(
            _seq(3, max_tokens=30))
    s = Scheduler(CacheManager(groups, 4, [16, 4], enable_prefix_caching=False), 4, 8, 64, (), "prefill_first")
    q = _seq(3, max_tokens=30)
    s.add(q)
    _run(s)
    assert q.finish_reason == "max_tokens" and q.num_completion_tokens == 30
    assert s.cache.pools[1].num_free == 4
    # a short answer never reaches the window's width: the same pool of 3 pages takes it
    Scheduler(CacheManager(groups, 4, [16, 3], enable_prefix_caching=False), 4, 8, 64, (), "prefill_first").add(
        _seq(3, max_tokens=4))
