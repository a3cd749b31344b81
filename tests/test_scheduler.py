"""The scheduler's decisions, on a real engine driven by plain torch ops on the CPU
(cases of qwen-server/src/engine.rs:1328-2529 that do not need a server)."""
import pytest

from cpu_engine import cpu_engine
from tiny_configs import random_ids
from tokenizer_amd.engine import (Failure, GenerateParams, Generated, QueueFull, Scheduler, SchedulerConfig,
                                  StopReason, generate)


def solo(folder, prompt, params):
    return generate(cpu_engine(folder), prompt, params)


def prompts(n, lengths, vocab=256):
    return [random_ids(vocab, lengths[i % len(lengths)], 40 + i) for i in range(n)]


def test_batched_equals_solo(model_folders):
    folder = model_folders["A"]
    engine = cpu_engine(folder, num_pages=64, max_requests=8)
    sched = Scheduler(engine, SchedulerConfig(max_batch_size=8, num_blocks=64))
    budgets = [5, 1, 4, 5, 2, 5, 3, 5]
    ps = prompts(8, [1, 2, 3, 4, 5, 6, 17, 31])
    ids = [sched.add_request(p, GenerateParams.greedy(n)) for p, n in zip(ps, budgets)]
    results = sched.run()
    for rid, prompt, n in zip(ids, ps, budgets):
        want = solo(folder, prompt, GenerateParams.greedy(n))
        assert isinstance(results[rid], Generated)
        assert results[rid].tokens == want.tokens and results[rid].reason == StopReason.MaxTokens
        assert results[rid].completion_tokens == n
    assert sched.stats.requests_finished == 8 and sched.stats.max_running == 8
    # The first iteration holds all eight prompts; later ones only single tokens of those still decoding.
    assert sorted(engine.forwards[0]) == sorted(len(p) for p in ps)
    assert all(set(step) == {1} for step in engine.forwards[1:])
    assert [len(step) for step in engine.forwards[1:]] == [7, 6, 5, 4]
    sched.assert_idle()


def test_warm_requests_in_a_batch_draw_as_they_would_alone(model_folders):
    folder = model_folders["A"]
    sched = Scheduler(cpu_engine(folder), SchedulerConfig())
    ps = prompts(3, [4, 9, 2])
    params = [GenerateParams(max_tokens=12, temperature=1.3, top_p=0.95, seed=s) for s in (5, 6, 5)]
    ids = [sched.add_request(p, q) for p, q in zip(ps, params)]
    results = sched.run()
    for rid, prompt, q in zip(ids, ps, params):
        assert results[rid].tokens == solo(folder, prompt, q).tokens
    sched.assert_idle()


def test_warm_requests_decode_in_bursts_and_draw_as_they_would_alone(model_folders):
    """Requests that draw with a temperature decode in bursts too, a greedy one among them (`Engine.decode_sampled`:
    the draws stay on the device, each drawing request's generator gives one uniform number for every step that is
    launched); one of them ends early on an end-of-sequence id in the middle of a burst, and every one gets the
    tokens it gets alone."""
    folder = model_folders["B"]
    engine = cpu_engine(folder, bursts=True)
    runs = []
    inner = engine.decode_sampled
    engine.decode_sampled = lambda rids, tokens, n_steps, draw, on_step=None: (
        runs.append((len(rids), n_steps)), inner(rids, tokens, n_steps, draw, on_step))[1]
    sched = Scheduler(engine, SchedulerConfig(decode_burst=8))
    ps = prompts(4, [4, 9, 2, 6], vocab=384)
    params = [GenerateParams(max_tokens=21, temperature=1.3, top_p=0.95, seed=5),
              GenerateParams(max_tokens=30, temperature=0.7, top_p=1.0, seed=6),
              GenerateParams(max_tokens=17, temperature=1.0, top_p=0.6, seed=5),
              GenerateParams.greedy(25)]                      # a greedy one among them keeps its greedy picks
    alone = [solo(folder, p, q) for p, q in zip(ps, params)]
    params[1].eos = [alone[1].tokens[12]]                    # the second request ends where it first meets this id
    alone[1] = solo(folder, ps[1], params[1])
    assert alone[1].reason == StopReason.Eos and len(alone[1].tokens) <= 12
    ids = [sched.add_request(p, q) for p, q in zip(ps, params)]
    results = sched.run()
    for rid, want in zip(ids, alone):
        assert (results[rid].tokens, results[rid].reason) == (want.tokens, want.reason)
    assert runs and runs[0] == (4, 8) and any(count == 3 for count, _ in runs)     # bursts of all four, then of three
    sched.assert_idle()


def test_token_budget_cuts_prompts_and_decoding_goes_first(model_folders):
    folder = model_folders["A"]
    engine = cpu_engine(folder, num_pages=64)
    sched = Scheduler(engine, SchedulerConfig(max_num_batched_tokens=16, prefill_chunk=10))
    long_a, long_b, short = random_ids(256, 37, 1), random_ids(256, 23, 2), random_ids(256, 3, 3)
    first = sched.add_request(short, GenerateParams.greedy(6))
    sched.step()                                         # the short one is through its prompt
    a = sched.add_request(long_a, GenerateParams.greedy(3))
    b = sched.add_request(long_b, GenerateParams.greedy(3))
    results = sched.run()
    assert all(sum(step) <= 16 for step in engine.forwards)
    assert engine.forwards[0] == [3]
    assert engine.forwards[1] == [1, 10, 5]              # the decoding token first, then portions in order of arrival
    assert engine.forwards[2] == [1, 10, 5]
    assert max(max(step) for step in engine.forwards) == 10
    for rid, prompt, n in ((first, short, 6), (a, long_a, 3), (b, long_b, 3)):
        assert results[rid].tokens == solo(folder, prompt, GenerateParams.greedy(n)).tokens
    sched.assert_idle()


def test_prompts_first_holds_decoding_back_until_the_prompts_are_through(model_folders):
    """The reference's order within an iteration (new sequences are prefilled before the batched decode,
    qwen-server/src/engine.rs:788-805) under a token budget: portions of prompts take the budget, decoding
    sequences what is left of it; the tokens are the same as in the other order."""
    folder = model_folders["A"]
    engine = cpu_engine(folder, num_pages=64)
    sched = Scheduler(engine, SchedulerConfig(max_num_batched_tokens=16, prefill_chunk=10, prompts_first=True))
    long_a, long_b, short = random_ids(256, 37, 1), random_ids(256, 23, 2), random_ids(256, 3, 3)
    first = sched.add_request(short, GenerateParams.greedy(6))
    sched.step()                                         # the short one is through its prompt
    a = sched.add_request(long_a, GenerateParams.greedy(3))
    b = sched.add_request(long_b, GenerateParams.greedy(3))
    results = sched.run()
    assert all(sum(step) <= 16 for step in engine.forwards)
    assert engine.forwards[0] == [3]
    # 37 and 23 prompt tokens in portions of at most 10 under a budget of 16: the decoding request waits while
    # they fill the budget and joins in the step that leaves room (7 + 5 + its one token).
    assert engine.forwards[1:5] == [[10, 6], [10, 6], [10, 6], [7, 5, 1]]
    assert engine.forwards[5] == [1, 1, 1]               # all three decode together from here
    assert all(set(step) == {1} for step in engine.forwards[5:])
    for rid, prompt, n in ((first, short, 6), (a, long_a, 3), (b, long_b, 3)):
        assert results[rid].tokens == solo(folder, prompt, GenerateParams.greedy(n)).tokens
    sched.assert_idle()


def test_pages_run_out_the_newest_is_preempted_and_recomputed(model_folders):
    # Pool of 3 pages, two 16-token prompts, 4 tokens each: both need a second page once they decode.
    folder = model_folders["A"]
    engine = cpu_engine(folder, num_pages=3, max_requests=4)
    sched = Scheduler(engine, SchedulerConfig(num_blocks=3, prefix_cache=False))
    ps = prompts(2, [16])
    ids = [sched.add_request(p, GenerateParams.greedy(4)) for p in ps]
    results = sched.run()
    assert sched.stats.preemptions >= 1 and sched.stats.last_preempted_id == ids[1]
    for rid, prompt in zip(ids, ps):
        assert results[rid].tokens == solo(folder, prompt, GenerateParams.greedy(4)).tokens
        assert results[rid].completion_tokens == 4
    # The recomputation ran the prompt and the tokens sampled so far in one portion.
    assert any(n > 16 for step in engine.forwards for n in step)
    sched.assert_idle()


def test_a_prompt_that_can_never_fit_fails_and_the_next_runs(model_folders):
    folder = model_folders["A"]
    sched = Scheduler(cpu_engine(folder, num_pages=1, max_requests=2), SchedulerConfig(num_blocks=1, prefix_cache=False))
    big = sched.add_request(random_ids(256, 17, 1), GenerateParams.greedy(2))
    small_prompt = random_ids(256, 5, 2)
    small = sched.add_request(small_prompt, GenerateParams.greedy(2))
    results = sched.run()
    assert isinstance(results[big], Failure)
    assert results[big].message == "kv pool has 1 blocks of 16; this sequence needs 2"
    assert results[small].tokens == solo(folder, small_prompt, GenerateParams.greedy(2)).tokens
    # One that fits its prompt but outgrows the whole pool while decoding fails the same way.
    grow = sched.add_request(random_ids(256, 15, 3), GenerateParams.greedy(5))
    results = sched.run()
    assert isinstance(results[grow], Failure) and "needs 2" in results[grow].message
    sched.assert_idle()


def test_a_sequence_that_outgrows_the_pool_alone_in_the_batch_does_not_take_the_next_with_it(model_folders):
    """Batches of one: the running sequence outgrows the whole pool and fails in an iteration that runs nothing.
    Its pages are back then, and the queue's front, which needs exactly the whole pool, runs in the next one
    (that nothing ran while nothing is running does not mean that the front can never be admitted)."""
    folder = model_folders["A"]
    config = SchedulerConfig(max_batch_size=1, num_blocks=5, prefix_cache=False, prefill_chunk=5,
                             max_num_batched_tokens=16)
    sched = Scheduler(cpu_engine(folder, num_pages=5, max_requests=1), config)
    outgrows = sched.add_request(random_ids(256, 80, 1), GenerateParams.greedy(9))     # 89 tokens: six pages
    fits_prompt = random_ids(256, 64, 2)
    fits = sched.add_request(fits_prompt, GenerateParams.greedy(9))                    # 73 tokens: five pages
    while sched.has_work():                      # one iteration a call, as a server's loop drives it
        sched.run(max_steps=1)
    results = sched.finished
    assert isinstance(results[outgrows], Failure) and "needs 6" in results[outgrows].message
    assert isinstance(results[fits], Generated), results[fits]
    assert results[fits].tokens == solo(folder, fits_prompt, GenerateParams.greedy(9)).tokens
    sched.assert_idle()


def test_requests_that_cannot_be_accepted(model_folders):
    sched = Scheduler(cpu_engine(model_folders["A"]), SchedulerConfig(max_waiting=2))
    empty = sched.add_request([], GenerateParams.greedy(3))
    assert sched.finished[empty].message == "prompt encoded to no tokens"
    too_long = sched.add_request(random_ids(256, 100, 1), GenerateParams.greedy(29))     # max_position_embeddings 128
    assert "exceeds max_position_embeddings 128" in sched.finished[too_long].message
    bad = sched.add_request([1, 2], GenerateParams(temperature=-1.0))
    assert "negative" in sched.finished[bad].message
    sched.add_request([1], GenerateParams.greedy(1))
    sched.add_request([2], GenerateParams.greedy(1))
    with pytest.raises(QueueFull):
        sched.add_request([3], GenerateParams.greedy(1))
    sched.run()
    sched.assert_idle()


def test_admission_is_first_in_first_out(model_folders):
    # The big request at the front waits for pages; the small one behind it must not overtake.
    folder = model_folders["A"]
    engine = cpu_engine(folder, num_pages=4, max_requests=4)
    sched = Scheduler(engine, SchedulerConfig(num_blocks=4, prefix_cache=False))
    running = sched.add_request(random_ids(256, 30, 1), GenerateParams.greedy(3))
    sched.step()
    big = sched.add_request(random_ids(256, 40, 2), GenerateParams.greedy(2))      # 3 pages, only 2 free
    small = sched.add_request(random_ids(256, 4, 3), GenerateParams.greedy(2))
    sched.step()
    assert [seq.id for seq in sched.running] == [running] and [seq.id for seq in sched.waiting] == [big, small]
    results = sched.run()
    assert all(isinstance(results[r], Generated) for r in (running, big, small))
    sched.assert_idle()


def test_a_request_joins_while_others_run(model_folders):
    folder = model_folders["A"]
    sched = Scheduler(cpu_engine(folder), SchedulerConfig())
    p1, p2 = random_ids(256, 7, 1), random_ids(256, 11, 2)
    first = sched.add_request(p1, GenerateParams.greedy(8))
    for _ in range(3):
        sched.step()
    second = sched.add_request(p2, GenerateParams.greedy(4))
    results = sched.run()
    assert results[first].tokens == solo(folder, p1, GenerateParams.greedy(8)).tokens
    assert results[second].tokens == solo(folder, p2, GenerateParams.greedy(4)).tokens
    sched.assert_idle()


def test_shared_prefix_is_reused_and_gives_the_same_tokens(model_folders):
    folder = model_folders["A"]
    prefix = random_ids(256, 48, 9)
    ps = [prefix + random_ids(256, 5 + i, 20 + i) for i in range(3)]

    def run(prefix_cache):
        engine = cpu_engine(folder, num_pages=32, prefix_cache=prefix_cache)
        sched = Scheduler(engine, SchedulerConfig(max_batch_size=2, num_blocks=32, prefix_cache=prefix_cache))
        ids = [sched.add_request(p, GenerateParams.greedy(4)) for p in ps]
        results = sched.run()
        sched.assert_idle()
        return [results[i].tokens for i in ids], engine.forwards, sched.stats

    with_cache, forwards_on, stats_on = run(True)
    without, forwards_off, stats_off = run(False)
    assert with_cache == without
    for prompt, tokens in zip(ps, with_cache):
        assert tokens == solo(folder, prompt, GenerateParams.greedy(4)).tokens
    # The third request starts after the first has published its pages: it runs only its own tail.
    assert sum(map(sum, forwards_on)) == sum(map(sum, forwards_off)) - 48
    assert stats_on.peak_blocks <= stats_off.peak_blocks


def test_cancel(model_folders):
    sched = Scheduler(cpu_engine(model_folders["A"]), SchedulerConfig())
    rid = sched.add_request([1, 2, 3], GenerateParams.greedy(10))
    waiting = sched.add_request([4, 5], GenerateParams.greedy(10))
    sched.step()
    sched.step()
    sched.cancel(rid)
    assert sched.finished[rid].reason == StopReason.Cancelled and len(sched.finished[rid].tokens) == 2
    sched.cancel(waiting)
    sched.run()
    sched.assert_idle()


@pytest.mark.parametrize("seed", range(6))
def test_requests_cancelled_at_random_keep_what_they_sampled(model_folders, seed):
    """Requests cancelled from outside at random iterations (waiting, in the middle of their prompt, decoding) or by
    their own chunk callback after so many chunks, among requests that run to their end, under small pools: a
    cancelled request holds a beginning of what it would have got alone, the others all of it, nothing is left."""
    import random
    from tokenizer_amd.engine.generate import Control
    rng = random.Random(3000 + seed)
    folder = model_folders["A"]
    num_pages = rng.choice([5, 8, 12, 30])
    config = SchedulerConfig(max_batch_size=rng.choice([1, 2, 4]), num_blocks=num_pages, prefix_cache=rng.random() < 0.5,
                             max_num_batched_tokens=rng.choice([8, 24, 64]), prefill_chunk=rng.choice([None, 7, 16]))
    engine = cpu_engine(folder, bursts=True, num_pages=num_pages, max_requests=config.max_batch_size,
                        prefix_cache=config.prefix_cache, counting=False)
    sched = Scheduler(engine, config)
    token_bytes = lambda token: bytes([97 + token % 7])
    shared = random_ids(256, 40, 7000 + seed)
    ids = {}
    for i in range(rng.randint(4, 7)):
        prompt = random_ids(256, rng.choice([1, 3, 15, 16, 17, 31, 40]), 50 * seed + i)
        if rng.random() < 0.4:
            prompt = shared[:rng.choice([16, 32, 40])] + prompt
        params = GenerateParams(max_tokens=rng.choice([1, 5, 9, 14]), temperature=rng.choice([0.0, 1.0]), seed=i)
        limit = rng.choice([None, None, 0, 1, 3])          # the callback says Stop after so many chunks

        def on_chunk(text, limit=limit, seen=[0]):
            if limit is None or (text == "" and limit > 0):
                return Control.Continue
            seen[0] += 1
            return Control.Stop if seen[0] > limit else Control.Continue

        ids[sched.add_request(prompt, params, token_bytes=token_bytes, on_chunk=on_chunk)] = (prompt, params, limit)
    from_outside = {rid: rng.randint(0, 12) for rid in ids if rng.random() < 0.3}
    step = 0
    while sched.has_work():
        for rid, when in from_outside.items():
            if when == step:
                sched.cancel(rid)
        sched.run(max_steps=1)
        step += 1
        assert step < 3000
        engine.cache.check_invariants()
    for rid, (prompt, params, limit) in ids.items():
        got = sched.finished[rid]
        assert isinstance(got, Generated), got
        want = generate(cpu_engine(folder), prompt, params, token_bytes=token_bytes)
        assert got.tokens == want.tokens[:len(got.tokens)]
        if got.reason == StopReason.Cancelled:
            assert rid in from_outside or limit is not None
        else:
            assert (got.tokens, got.text, got.reason) == (want.tokens, want.text, want.reason)
    sched.assert_idle()


@pytest.mark.parametrize("prompts_first", [False, True])
@pytest.mark.parametrize("seed", range(12))
def test_random_arrivals_pools_and_budgets_give_solo_results(model_folders, seed, prompts_first):
    """Random prompts, output lengths, pool sizes, batch caps, token budgets, portion sizes and arrival times
    (shared prefixes included), under either order of prompts and decoding: whatever the scheduler decides, every
    request gets the tokens it would get alone, and when all is over no page, count or slot is left."""
    import random
    rng = random.Random(seed)
    folder = model_folders["A"]
    page = 16
    num_pages = rng.choice([4, 5, 6, 9, 24])
    config = SchedulerConfig(max_batch_size=rng.choice([1, 2, 3, 5]), num_blocks=num_pages,
                             prefix_cache=rng.random() < 0.5, max_num_batched_tokens=rng.choice([8, 16, 40]),
                             prefill_chunk=rng.choice([None, 5, 16]), max_waiting=64, prompts_first=prompts_first)
    engine = cpu_engine(folder, bursts=True, num_pages=num_pages, max_requests=config.max_batch_size,
                        prefix_cache=config.prefix_cache)
    sched = Scheduler(engine, config)
    shared = random_ids(256, 35, 900 + seed)
    plan = []
    for i in range(rng.randint(4, 9)):
        prompt = random_ids(256, rng.choice([1, 2, 7, 16, 17, 33, 48]), 100 * seed + i)
        if rng.random() < 0.4:
            prompt = shared[:rng.choice([16, 32, 35])] + prompt
        plan.append((rng.randint(0, 6), prompt, rng.randint(0, 9)))
    ids, step = {}, 0
    pending = sorted(plan, key=lambda item: item[0])
    while pending or sched.has_work():
        while pending and pending[0][0] <= step:
            _, prompt, n = pending.pop(0)
            ids[sched.add_request(prompt, GenerateParams.greedy(n))] = (prompt, n)
        if sched.has_work():
            sched.run(max_steps=1)
        step += 1
        assert step < 2000
        engine.cache.check_invariants()
    assert all(sum(tokens) <= config.max_num_batched_tokens for tokens in engine.forwards)
    for rid, (prompt, n) in ids.items():
        result = sched.finished[rid]
        if isinstance(result, Failure):
            # Only a sequence that the whole pool cannot hold may fail, and it says so.
            assert "kv pool has" in result.message and -(-(len(prompt) + n) // page) > num_pages
            continue
        assert result.tokens == solo(folder, prompt, GenerateParams.greedy(n)).tokens, (rid, len(prompt), n)
    sched.assert_idle()


def requests_of_every_kind(rng, vocab, seed):
    """Prompts (some with a shared beginning) with greedy or warm sampling, nucleus cuts, end-of-sequence ids, stop
    strings and budgets down to zero, and the steps at which they arrive."""
    shared = random_ids(vocab, 40, 7000 + seed)
    plan = []
    for i in range(rng.randint(3, 8)):
        prompt = random_ids(vocab, rng.choice([1, 3, 15, 16, 17, 31, 40]), 50 * seed + i)
        if rng.random() < 0.4:
            prompt = shared[:rng.choice([16, 32, 40])] + prompt
        warm = rng.random() < 0.5
        params = GenerateParams(max_tokens=rng.choice([0, 1, 2, 5, 9, 14]),
                                temperature=rng.choice([0.7, 1.0, 1.5]) if warm else 0.0,
                                top_p=rng.choice([1.0, 0.9, 0.5]) if warm else 1.0, seed=rng.randint(0, 99),
                                eos=[rng.randrange(vocab) for _ in range(rng.choice([0, 0, 3, 40]))],
                                stop=rng.choice([[], [], ["ab"], ["cc", "gfe"], ["a"]]))
        plan.append((rng.randint(0, 5), prompt, params))
    return sorted(plan, key=lambda item: item[0])


def run_requests_of_every_kind(make_engine, folder, vocab, seed, prompts_first=False):
    """Drive a scheduler over `make_engine(...)` with random limits through such requests; every result must be
    what the same request gives when it is generated alone."""
    import random
    rng = random.Random(1000 + seed)
    num_pages = rng.choice([5, 6, 8, 12, 30])
    config = SchedulerConfig(max_batch_size=rng.choice([1, 2, 4, 6]), num_blocks=num_pages,
                             prefix_cache=rng.random() < 0.5, max_num_batched_tokens=rng.choice([8, 24, 64]),
                             prefill_chunk=rng.choice([None, 7, 16]), max_waiting=64,
                             decode_burst=rng.choice([1, 4, 16]), prompts_first=prompts_first)
    engine = make_engine(folder, num_pages=num_pages, max_requests=config.max_batch_size,
                         prefix_cache=config.prefix_cache)
    alone = make_engine(folder, num_pages=40, max_requests=1, prefix_cache=False)
    sched = Scheduler(engine, config)
    token_bytes = lambda token: bytes([97 + token % 7])
    pending = requests_of_every_kind(rng, vocab, seed)
    ids, step = {}, 0
    while pending or sched.has_work():
        while pending and pending[0][0] <= step:
            _, prompt, params = pending.pop(0)
            ids[sched.add_request(prompt, params, token_bytes=token_bytes)] = (prompt, params)
        if sched.has_work():
            sched.run(max_steps=1)
        step += 1
        assert step < 3000
        engine.cache.check_invariants()
    for rid, (prompt, params) in ids.items():
        got = sched.finished[rid]
        if isinstance(got, Failure):
            assert "kv pool has" in got.message and -(-(len(prompt) + params.max_tokens) // 16) > num_pages
            continue
        want = generate(alone, prompt, params, token_bytes=token_bytes)
        assert (got.tokens, got.text, got.reason, got.completion_tokens, "".join(got.chunks)) == \
               (want.tokens, want.text, want.reason, want.completion_tokens, "".join(want.chunks)), (rid, params)
    sched.assert_idle()


@pytest.mark.parametrize("prompts_first", [False, True])
@pytest.mark.parametrize("seed", range(8))
def test_requests_of_every_kind_get_what_they_get_alone(model_folders, seed, prompts_first):
    """Greedy and warm requests, nucleus cuts, end-of-sequence ids, stop strings and zero budgets side by side, under
    random pools, batch caps, token budgets and portion sizes, decoding or prompts first: tokens, text, chunks,
    reason and counts of every request equal those of the request generated alone
    (qwen-server/src/engine.rs:1328-1420 widened)."""
    name = "ABC"[seed % 3]
    vocab = {"A": 256, "B": 384, "C": 320}[name]
    run_requests_of_every_kind(lambda folder, **kw: cpu_engine(folder, counting=False, bursts=True, **kw), model_folders[name],
                               vocab, seed, prompts_first)


def test_a_step_that_may_not_reserve_refuses_an_entry_without_pages(model_folders):
    """The scheduler reserves while it plans; the step it then runs takes nothing from the pool."""
    from tokenizer_amd.engine import StepEntry
    engine = cpu_engine(model_folders["A"], num_pages=4, counting=False)
    engine.add_request("a")
    with pytest.raises(RuntimeError, match="too few pages"):
        engine.step([StepEntry("a", [1, 2, 3], [2])], reserve=False)
    assert engine.cache.seq_len("a") == 0 and engine.cache.groups[0].allocator.live_count() == 0
    assert engine.cache.reserve("a", 3)
    assert engine.step([StepEntry("a", [1, 2, 3], [2])], reserve=False).shape == (1, 256)
    assert engine.cache.seq_len("a") == 3 and engine.cache.groups[0].allocator.live_count() == 1
    engine.end_request("a")


@pytest.mark.parametrize("page_size", [16, 48, 128])
def test_a_pool_made_for_so_many_tokens_holds_them_at_any_page_size(model_folders, page_size):
    """`Engine(max_tokens=N)`: N counts each live request's tokens rounded up to a multiple of 64.  Pages that do
    not divide 64 round each request up on their own; four requests of 64 tokens still find their pages."""
    from kernel_refs import PlainOps
    from tokenizer_amd.engine import Engine, load_model
    engine = Engine(load_model(model_folders["A"], "float32", "cpu", ops=PlainOps()), max_tokens=4 * 64,
                    page_size=page_size, max_requests=4)
    for rid in range(4):
        engine.add_request(rid)
        assert engine.cache.reserve(rid, 64), (rid, engine.cache.num_pages)
    for rid in range(4):
        engine.end_request(rid)
    engine.cache.check_invariants()


def test_a_burst_the_pool_cannot_hold_is_shortened_instead_of_taking_pages_early(model_folders):
    """Three sequences decode side by side in a pool that cannot hold all of them to their ends: sooner or later one
    is preempted.  A burst of sixteen steps asks for the pages of all of them together and is halved until the pool
    can hold it; it never leaves some sequences with pages they do not need yet while another finds none for its
    next token.  So bursts preempt no more often, and forward no more tokens again, than single steps do, and give
    the same tokens."""
    folder = model_folders["A"]
    prompts = [random_ids(256, n, 400 + i) for i, n in enumerate([15, 9, 30])]
    stats = {}
    for burst in (1, 16):
        engine = cpu_engine(folder, bursts=True, num_pages=7, max_requests=3, counting=False)
        sched = Scheduler(engine, SchedulerConfig(max_batch_size=3, num_blocks=7, prefix_cache=False, decode_burst=burst))
        ids = [sched.add_request(prompt, GenerateParams.greedy(24)) for prompt in prompts]
        results = sched.run()
        for rid, prompt in zip(ids, prompts):
            assert results[rid].tokens == solo(folder, prompt, GenerateParams.greedy(24)).tokens
        sched.assert_idle()
        stats[burst] = sched.stats
    assert stats[1].preemptions >= 1                                   # the pool is too small for all of them
    assert stats[16].preemptions <= stats[1].preemptions
    assert stats[16].tokens_forwarded <= stats[1].tokens_forwarded
    # With room for everything the bursts run at full length: far fewer iterations of the scheduler than tokens.
    engine = cpu_engine(folder, bursts=True, num_pages=12, max_requests=3, counting=False)
    sched = Scheduler(engine, SchedulerConfig(max_batch_size=3, num_blocks=12, prefix_cache=False, decode_burst=16))
    ids = [sched.add_request(prompt, GenerateParams.greedy(20)) for prompt in prompts]
    steps = 0
    while sched.has_work():
        sched.run(max_steps=1)
        steps += 1
    assert steps <= 8 and sched.stats.preemptions == 0
    for rid, prompt in zip(ids, prompts):
        assert sched.finished[rid].tokens == solo(folder, prompt, GenerateParams.greedy(20)).tokens
