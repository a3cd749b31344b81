"""The scheduler on the device: preemption with recomputation, shared prefix pages, prompts cut into portions
whose shape recurs (so that captured graphs replay them), against the plain implementation's tokens."""
import pytest
import torch

from plain import qwen2_plain as plain
from tiny_configs import TINY, random_ids

pytestmark = pytest.mark.gpu


def engine_for(folder, dtype, **kw):
    from tokenizer_amd.engine import Engine, load_model
    return Engine(load_model(folder, dtype), **kw)


def check_greedy(cfg, tensors, prompt, tokens, dtype, n_tokens):
    """The tokens a greedy request produced, against the plain implementation.  float32: the same ids.
    bfloat16: rounding may pick another of two nearly equal logits, after which the sequences differ for good;
    so every token is checked against the plain logits of the sequence the engine itself went along: it must
    be the maximum of its row up to what bfloat16 rounding can move a logit."""
    assert len(tokens) == n_tokens
    if dtype == "float32":
        assert tokens == plain.greedy_generate(cfg, tensors, prompt, n_tokens)
        return
    logits = plain.all_logits(cfg, tensors, list(prompt) + list(tokens))
    for k, token in enumerate(tokens):
        row = logits[len(prompt) - 1 + k]
        assert float(row.max() - row[token]) <= 4e-2 * max(1.0, float(row.abs().max())), (k, token)


@pytest.mark.parametrize("dtype, prompts_first", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_few_pages_a_shared_prefix_and_portions_on_the_device(model_folders, dtype, prompts_first):
    """Six requests, three of which start with the same 40 tokens, through a pool of eight pages with prompts cut
    into portions of sixteen: some are preempted and recomputed, the later sharers take over the prefix's pages,
    decode steps and recurring portion shapes replay captured graphs.  Every request gets the plain
    implementation's tokens, and nothing is left over.  (Cases of qwen-server/src/engine.rs:1833-1908,
    1965-2320 and 2470-2529, run on the kernels.)"""
    from tokenizer_amd.engine import Generated, GenerateParams, Scheduler, SchedulerConfig
    name = "B"
    cfg, tensors = plain.load_folder(model_folders[name])
    vocab = cfg["vocab_size"]
    prefix = random_ids(vocab, 40, 7)
    prompts = [prefix + random_ids(vocab, 6, 1), random_ids(vocab, 21, 2), prefix + random_ids(vocab, 9, 3),
               random_ids(vocab, 33, 4), prefix + random_ids(vocab, 3, 5), random_ids(vocab, 17, 6)]
    eng = engine_for(model_folders[name], dtype, num_pages=8, max_requests=3, prefix_cache=True)
    eng.pools.poison()
    sched = Scheduler(eng, SchedulerConfig(max_batch_size=3, num_blocks=8, prefix_cache=True, prefill_chunk=16,
                                           max_num_batched_tokens=48, prompts_first=prompts_first))
    rids = [sched.add_request(p, GenerateParams.greedy(12)) for p in prompts]
    results = sched.run()
    for rid, prompt in zip(rids, prompts):
        assert isinstance(results[rid], Generated), results[rid]
        check_greedy(cfg, tensors, prompt, results[rid].tokens, dtype, 12)
    assert sched.stats.preemptions >= 1 and sched.stats.prefix_hits >= 2 and sched.stats.prefix_tokens_reused >= 64
    assert eng.use_graphs and eng.graphs
    sched.assert_idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_long_prompts_replay_graphs_narrower_than_their_tables(tmp_path, dtype):
    """Prompts longer than a graph's context bucket, one after another, cut into equal portions: the pages of a
    whole prompt are reserved at admission, so during its first portions a request's block table is wider than
    the table of the graph that the recurring shape replays.  Tokens with graphs equal tokens without, and the
    plain implementation's."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig
    raw = dict(TINY["A"][0], max_position_embeddings=2048, sliding_window=2048)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 21, str(tmp_path / "long"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    prompts = [random_ids(raw["vocab_size"], 1100, 300 + i) for i in range(4)]
    tokens = {}
    for use_graphs in (True, False):
        eng = engine_for(folder, dtype, num_pages=80, max_requests=1, use_graphs=use_graphs)
        eng.pools.poison()
        sched = Scheduler(eng, SchedulerConfig(max_batch_size=1, num_blocks=80, prefix_cache=False, prefill_chunk=256,
                                               max_num_batched_tokens=256))
        rids = [sched.add_request(p, GenerateParams.greedy(6)) for p in prompts]
        results = sched.run()
        tokens[use_graphs] = [results[rid].tokens for rid in rids]
        if use_graphs:
            portion_graphs = [key for key in eng.graphs if not isinstance(key[0], int)]
            assert portion_graphs, "no portion shape was captured"
            # The first portions replay graphs for contexts of 512 tokens: 32 pages, where the request holds 69.
            assert any(eng.graphs[key].width < 69 for key in portion_graphs)
        sched.assert_idle()
    if dtype == "float32":        # (bfloat16 portions of this many rows go to different products when recorded)
        assert tokens[True] == tokens[False]
    for use_graphs in (True, False):
        for prompt, got in zip(prompts, tokens[use_graphs]):
            check_greedy(cfg, tensors, prompt, got, dtype, 6)


def test_a_shared_prefix_under_replayed_graphs_with_heads_of_128_in_groups_of_seven(tmp_path):
    """Twelve requests that begin with the same 320 tokens, at the head shapes of the 7B model (28 query heads of
    128 over 4 key heads, a width of 3,584, beyond what the fused products normalise themselves), in bfloat16
    with the prefix cache: the first request's pages serve the others, whose remaining tokens run as portions
    beside decoded tokens, and decode steps and recurring portions replay captured graphs.  In the second pass
    over the same requests nearly every step is a replay.  In both passes every token is the plain
    implementation's choice on the sequence the engine went along (the passes' tokens need not be equal: a
    product of a recorded step may be another kernel's than the same product launched eagerly, and round
    differently)."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import Generated, GenerateParams, Scheduler, SchedulerConfig
    raw = dict(TINY["A"][0], num_hidden_layers=2, vocab_size=600, max_position_embeddings=512, sliding_window=512,
               tie_word_embeddings=False, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
               intermediate_size=640)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 31, str(tmp_path / "heads128"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    shared = random_ids(600, 320, 70)
    prompts = [shared + random_ids(600, 9 + 5 * i, 71 + i) for i in range(12)]
    pages = sum(-(-(len(p) + 20) // 16) for p in prompts) + 8
    eng = engine_for(folder, "bfloat16", num_pages=pages, max_requests=12, prefix_cache=True)
    eng.pools.poison()
    passes = []
    for _ in range(2):
        sched = Scheduler(eng, SchedulerConfig(max_batch_size=12, num_blocks=pages, prefix_cache=True,
                                               max_num_batched_tokens=128))
        rids = [sched.add_request(prompts[0], GenerateParams.greedy(20))]
        sched.step()                          # the first prompt's first portion is cached when the others arrive
        sched.step()
        sched.step()
        rids += [sched.add_request(p, GenerateParams.greedy(20)) for p in prompts[1:]]
        before = (eng.steps, eng.steps_replayed)
        results = sched.run()
        assert all(isinstance(results[rid], Generated) for rid in rids)
        assert sched.stats.prefix_hits >= 11 and sched.stats.prefix_tokens_reused >= 11 * 304
        passes.append(([results[rid].tokens for rid in rids], eng.steps - before[0], eng.steps_replayed - before[1]))
        sched.assert_idle()
    assert passes[1][2] >= passes[1][1] - 6, "the second pass should replay nearly every step"
    for got, _, _ in passes:
        for prompt, tokens in zip(prompts, got):
            check_greedy(cfg, tensors, prompt, tokens, "bfloat16", 20)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_back_to_back_give_what_single_steps_give(model_folders, dtype):
    """Greedy decoding runs in bursts of steps whose ids stay on the device (the host reads them one step late).
    A sequence that meets its end-of-sequence id, or a stop string, in the middle of a burst ends there, the
    others keep the token of the step that was already under way, and every request gets what it gets with one
    step at a time."""
    from tokenizer_amd.engine import Generated, GenerateParams, Scheduler, SchedulerConfig, StopReason
    name = "B"
    cfg, tensors = plain.load_folder(model_folders[name])
    vocab = cfg["vocab_size"]
    prompts = [random_ids(vocab, n, 500 + n) for n in (7, 19, 33, 4, 12)]
    budgets = [40, 25, 40, 9, 33]
    want = [plain.greedy_generate(cfg, tensors, p, n) for p, n in zip(prompts, budgets)]
    # An id that the first request meets for the first time some steps in: it ends there; others may meet it too.
    ends_at = next(j for j in range(5, 40) if want[0][j] not in want[0][:j])
    eos = want[0][ends_at]
    token_bytes = lambda token: bytes([65 + token % 26])
    stop = bytes([65 + want[2][20] % 26, 65 + want[2][21] % 26]).decode()    # two letters the third request spells

    def run(burst):
        eng = engine_for(model_folders[name], dtype, num_pages=40, max_requests=4)
        eng.pools.poison()
        sched = Scheduler(eng, SchedulerConfig(max_batch_size=4, num_blocks=40, prefix_cache=False, decode_burst=burst))
        rids = []
        for i, (prompt, budget) in enumerate(zip(prompts, budgets)):
            params = GenerateParams.greedy(budget)
            params.eos = [eos]
            if i == 2:
                params.stop = [stop]
            rids.append(sched.add_request(prompt, params, token_bytes=token_bytes))
        results = sched.run()
        sched.assert_idle()
        return [results[rid] for rid in rids], sched.stats

    bursts, stats = run(16)
    singles, single_stats = run(1)
    assert stats.steps == single_stats.steps or dtype == "bfloat16"
    for i, (a, b) in enumerate(zip(bursts, singles)):
        assert isinstance(a, Generated) and isinstance(b, Generated)
        if dtype == "float32":
            assert (a.tokens, a.reason, a.text, a.completion_tokens) == (b.tokens, b.reason, b.text, b.completion_tokens), i
            cut = want[i].index(eos) if eos in want[i] else len(want[i])
            assert a.tokens[:cut] == want[i][:len(a.tokens[:cut])] and len(a.tokens) <= cut
    if dtype == "float32":
        assert bursts[0].reason == StopReason.Eos and len(bursts[0].tokens) == ends_at
        assert bursts[2].reason in (StopReason.StopString, StopReason.Eos)
        assert any(r.reason == StopReason.MaxTokens for r in bursts)


@pytest.mark.parametrize("seed, prompts_first", [(0, False), (1, False), (2, False), (3, True), (4, True), (5, True)])
def test_random_arrivals_pools_and_budgets_on_the_device(model_folders, seed, prompts_first):
    """Random prompts (some with a shared beginning), output lengths, pool sizes, batch caps, token budgets,
    portion sizes, burst lengths and arrival times, decoding requests or prompts first, in float32 on the kernels
    with graphs: whatever the scheduler decides, every request gets the plain implementation's tokens, and in the
    end nothing is left over."""
    import random
    from tokenizer_amd.engine import Failure, GenerateParams, Scheduler, SchedulerConfig
    rng = random.Random(seed)
    name = "B"
    cfg, tensors = plain.load_folder(model_folders[name])
    vocab, page = cfg["vocab_size"], 16
    num_pages = rng.choice([5, 7, 10, 24])
    config = SchedulerConfig(max_batch_size=rng.choice([1, 2, 3, 5]), num_blocks=num_pages,
                             prefix_cache=rng.random() < 0.5, max_num_batched_tokens=rng.choice([8, 16, 40]),
                             prefill_chunk=rng.choice([None, 5, 16]), max_waiting=64,
                             decode_burst=rng.choice([1, 3, 16]), prompts_first=prompts_first)
    eng = engine_for(model_folders[name], "float32", num_pages=num_pages, max_requests=config.max_batch_size,
                     prefix_cache=config.prefix_cache)
    eng.pools.poison()
    sched = Scheduler(eng, config)
    shared = random_ids(vocab, 35, 900 + seed)
    plan = []
    for i in range(rng.randint(4, 8)):
        prompt = random_ids(vocab, rng.choice([1, 2, 7, 16, 17, 33, 48]), 100 * seed + i)
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
        eng.cache.check_invariants()
    for rid, (prompt, n) in ids.items():
        result = sched.finished[rid]
        if isinstance(result, Failure):
            assert "kv pool has" in result.message and -(-(len(prompt) + n) // page) > num_pages
            continue
        assert result.tokens == plain.greedy_generate(cfg, tensors, prompt, n), (rid, len(prompt), n)
    sched.assert_idle()


@pytest.mark.parametrize("seed", range(8, 24))
def test_requests_of_every_kind_on_the_device(model_folders, seed):
    """The host-side test of the same name on the kernels, in float32 with graphs, bursts of decode steps and
    draws on the device (the later seeds with prompts before decoding): every request gets what it gets alone."""
    from test_scheduler import run_requests_of_every_kind
    name = "ABC"[seed % 3]
    vocab = {"A": 256, "B": 384, "C": 320}[name]
    run_requests_of_every_kind(lambda folder, **kw: engine_for(folder, "float32", **kw), model_folders[name], vocab, seed,
                               prompts_first=seed >= 16)
