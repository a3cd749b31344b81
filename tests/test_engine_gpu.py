"""The engine on the GPU against the plain implementation: whole prompts, decoding, portions, mixed batches."""
import pytest
import torch

from plain import qwen2_plain as plain
from tiny_configs import TINY, random_ids

pytestmark = pytest.mark.gpu

# float32: the reference's own tolerance between its paths is 1e-4 (qwen-infer/src/model.rs:1455-1531);
# logits here are of order 1.  bfloat16: rounding to 8 bits at every layer boundary, a few percent of the
# largest logit at most.
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


@pytest.fixture(scope="module")
def oracle(model_folders):
    cache = {}

    def get(name, ids):
        key = (name, tuple(ids))
        if key not in cache:
            cfg, tensors = plain.load_folder(model_folders[name])
            cache[key] = plain.all_logits(cfg, tensors, ids)
        return cache[key]
    return get


def engine_for(folder, dtype, **kw):
    from tokenizer_amd.engine import Engine, load_model
    return Engine(load_model(folder, dtype), **kw)


def close(got, want, dtype, tolerance=None):
    got = got.float().cpu()
    err = float((got - want).abs().max())
    scale = float(want.abs().max())
    bound = (TOL[dtype] if tolerance is None else tolerance) * max(scale, 1.0)
    assert err <= bound, f"max abs error {err} against logits up to {scale}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_whole_prompts(model_folders, oracle, name, dtype):
    from tokenizer_amd.engine import StepEntry
    vocab = TINY[name][0]["vocab_size"]
    eng = engine_for(model_folders[name], dtype, num_pages=16, max_requests=4)
    for seed, length in enumerate([1, 5, 17, 31, 64, 100]):
        ids = random_ids(vocab, length, seed)
        eng.add_request(seed)
        got = eng.step([StepEntry(seed, ids, list(range(length)))])
        close(got, oracle(name, ids), dtype)
        eng.end_request(seed)
    eng.cache.check_invariants()


import trace_tools as tt

LENGTHS = [1, 9, 40, 64, 100, 33, 77]


def requests_for(name):
    raw = TINY[name][0]
    lens = [min(n, raw["max_position_embeddings"]) for n in LENGTHS]
    return {f"r{i}": random_ids(raw["vocab_size"], n, 10 + i) for i, n in enumerate(lens)}


def check_trace(model_folders, oracle, name, dtype, steps):
    reqs = requests_for(name)
    eng = engine_for(model_folders[name], dtype, max_tokens=tt.peak_tokens(steps), max_requests=4)
    eng.pools.poison()          # a read of a slot no request wrote shows up as NaN
    got = tt.run_in_process(eng, steps)
    for rid, ids in reqs.items():
        close(got[rid], oracle(name, ids), dtype)
    eng.cache.check_invariants()
    assert not eng.cache.requests
    for group in eng.cache.groups:
        assert group.allocator.all_refcounts_zero()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_last_32_tokens_one_by_one(model_folders, oracle, name, dtype):
    check_trace(model_folders, oracle, name, dtype, tt.decode_tail(requests_for(name), 32))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_portions_of_changing_size(model_folders, oracle, name, dtype):
    check_trace(model_folders, oracle, name, dtype, tt.portions(requests_for(name), 3))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
@pytest.mark.parametrize("seed", [4, 5])
def test_mixed_batches_with_reused_pages(model_folders, oracle, name, dtype, seed):
    steps = tt.mixed(requests_for(name), seed)
    assert max(len(s["entries"]) for s in steps) >= 3
    check_trace(model_folders, oracle, name, dtype, steps)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding(model_folders, oracle, name, dtype):
    # Three tokens of prompt, then every further token alone up to the position limit of 256.
    raw = TINY[name][0]
    ids = random_ids(raw["vocab_size"], 256, 99)
    steps = tt.decode_tail({"long": ids}, tail=253)
    eng = engine_for(model_folders[name], dtype, max_tokens=256, max_requests=2)
    eng.pools.poison()
    got = tt.run_in_process(eng, steps)
    close(got["long"], oracle(name, ids), dtype)


_LONG_ORACLE: dict = {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_thousands_of_tokens_of_context(tmp_path, dtype):
    """A context far beyond the other tests' (5,200 tokens, a position limit of 8,192): the prompt in portions of
    2,048 and less beside a second request that decodes, then single tokens across an end of a decode graph's
    context bucket.  Page numbers, slots and key ranges are large here; two rows of the long request and every row
    of the short one are compared with the plain implementation."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import StepEntry
    raw = dict(TINY["A"][0], max_position_embeddings=8192, sliding_window=8192, rope_theta=1000000.0)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 11, str(tmp_path / "long"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    long_ids, short_ids = random_ids(256, 5200, 31), random_ids(256, 60, 32)
    if "long" not in _LONG_ORACLE:                                # the same weights for both dtypes: computed once
        _LONG_ORACLE["long"] = plain.all_logits(cfg, tensors, long_ids)
        _LONG_ORACLE["short"] = plain.all_logits(cfg, tensors, short_ids)
    want_long, want_short = _LONG_ORACLE["long"], _LONG_ORACLE["short"]
    eng = engine_for(folder, dtype, max_tokens=5200 + 64 + 64, max_requests=2)
    eng.pools.poison()
    eng.add_request("long"), eng.add_request("short")
    got_long, got_short = {}, {}
    at, short_at = 0, 0
    for portion in (2048, 2048, 1000, 3, 64):                     # 5,163 tokens in portions, the short one beside them
        entries = [StepEntry("long", long_ids[at:at + portion], [portion - 1])]
        take = 20 if short_at == 0 else 1
        entries.append(StepEntry("short", short_ids[short_at:short_at + take], list(range(take))))
        logits = eng.step(entries).float().cpu()
        got_long[at + portion - 1] = logits[0]
        for i in range(take):
            got_short[short_at + i] = logits[1 + i]
        at, short_at = at + portion, short_at + take
    while at < len(long_ids):                                      # single tokens, through position 5,120 = 10 x 512
        entries = [StepEntry("long", [long_ids[at]], [0])]
        if short_at < len(short_ids):
            entries.append(StepEntry("short", [short_ids[short_at]], [0]))
        logits = eng.step(entries).float().cpu()
        got_long[at] = logits[0]
        if short_at < len(short_ids):
            got_short[short_at] = logits[1]
            short_at += 1
        at += 1
    assert len(eng.graphs) >= 2 or not eng.use_graphs
    close(torch.stack([got_long[p] for p in sorted(got_long)]), want_long[sorted(got_long)], dtype)
    close(torch.stack([got_short[p] for p in sorted(got_short)]), want_short[sorted(got_short)], dtype)
    eng.end_request("long"), eng.end_request("short")
    eng.cache.check_invariants()


@pytest.mark.parametrize("heads,shape", [((28, 4, 128), 12), ((14, 2, 64), 11)])
def test_long_prompts_with_large_heads_through_the_engine(tmp_path, heads, shape):
    """28 query heads of 128 over 4 kv heads, or 14 of 64 over 2 (the head shapes of the 7B and the 0.5B model, two
    narrow layers), and prompts long enough that the launcher gives their portions to the prompt kernel whose waves
    share each block of keys: a prompt of 2,300 tokens in one step beside a short one, then a portion of 700 tokens
    that starts inside a page after 1,650 cached ones (fewer tiles: another shape of that kernel), then single
    tokens; also under a window of 1,000 keys in the upper layer.  Logits against the plain implementation."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import StepEntry
    from tokenizer_amd.kernels import get_ops
    ops = get_ops()
    assert ops.prefill_shared == 0
    n_q, n_kv, d = heads
    assert ops.lib.ta_prefill_attention_shared_plan(144 + 2, n_q, n_kv, d, 2560) == shape     # the first step below
    raw = dict(TINY["A"][0], num_hidden_layers=2, hidden_size=n_q * d, num_attention_heads=n_q, num_key_value_heads=n_kv,
               intermediate_size=256, vocab_size=300, max_position_embeddings=4096, rope_theta=1000000.0,
               use_sliding_window=True, sliding_window=1000, max_window_layers=1)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 17, str(tmp_path / "heads"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    a_ids, b_ids, c_ids = random_ids(300, 2310, 41), random_ids(300, 30, 42), random_ids(300, 2360, 43)
    want = {"a": plain.all_logits(cfg, tensors, a_ids), "b": plain.all_logits(cfg, tensors, b_ids),
            "c": plain.all_logits(cfg, tensors, c_ids)}
    eng = engine_for(folder, "bfloat16", max_tokens=2368 + 64 + 2368, max_requests=3)
    eng.pools.poison()
    for rid in "abc":
        eng.add_request(rid)
    rows = [0, 15, 16, 1000, 1001, 1650, 2299]
    logits = eng.step([StepEntry("a", a_ids[:2300], rows), StepEntry("b", b_ids[:25], [0, 24])]).float().cpu()
    close(logits[:len(rows)], want["a"][rows], "bfloat16")
    close(logits[len(rows):], want["b"][[0, 24]], "bfloat16")
    logits = eng.step([StepEntry("c", c_ids[:1650], [1649])]).float().cpu()
    close(logits, want["c"][[1649]], "bfloat16")
    logits = eng.step([StepEntry("c", c_ids[1650:2350], [0, 699]), StepEntry("a", a_ids[2300:2301], [0])]).float().cpu()
    close(logits[:2], want["c"][[1650, 2349]], "bfloat16")
    close(logits[2:], want["a"][[2300]], "bfloat16")
    for i in range(2301, 2310):
        logits = eng.step([StepEntry("a", a_ids[i:i + 1], [0]), StepEntry("c", c_ids[i + 49:i + 50], [0])]).float().cpu()
        close(logits[:1], want["a"][[i]], "bfloat16")
        close(logits[1:], want["c"][[i + 49]], "bfloat16")
    for rid in "abc":
        eng.end_request(rid)
    eng.cache.check_invariants()


@pytest.mark.parametrize("heads", [(28, 4, 128), (14, 2, 64)])
def test_short_portions_behind_a_long_context_through_the_engine(tmp_path, heads):
    """A prompt of 3,400 tokens: 3,000 in one step, then equal portions of 64 beside a decoded token of another
    request.  The portions are a handful of tiles with thousands of keys behind them, whose keys the prompt kernel
    cuts over workgroups (a second kernel merges the parts); their shape recurs, so the later ones replay a graph
    with those two kernels in it.  Every portion against the plain implementation, recorded and not."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import StepEntry
    from tokenizer_amd.kernels import get_ops
    n_q, n_kv, d = heads
    ops = get_ops()
    assert ops.lib.ta_prefill_attention_key_splits(4, n_q, n_kv, d, -1, 0, 3100, 0, 0) > 1       # the portions below
    raw = dict(TINY["A"][0], num_hidden_layers=2, hidden_size=n_q * d, num_attention_heads=n_q, num_key_value_heads=n_kv,
               intermediate_size=256, vocab_size=300, max_position_embeddings=4096, rope_theta=1000000.0)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 23, str(tmp_path / "far"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    a_ids, b_ids = random_ids(300, 3400, 81), random_ids(300, 40, 82)
    want_a, want_b = plain.all_logits(cfg, tensors, a_ids), plain.all_logits(cfg, tensors, b_ids)
    got = {}
    for use_graphs in (True, False):
        eng = engine_for(folder, "bfloat16", max_tokens=3456 + 64, max_requests=2, use_graphs=use_graphs)
        eng.pools.poison()
        eng.add_request("a")
        eng.add_request("b")
        eng.step([StepEntry("a", a_ids[:3000], []), StepEntry("b", b_ids[:30], [])])
        for k in range(6):
            at = 3000 + 64 * k
            logits = eng.step([StepEntry("a", a_ids[at:at + 64], [0, 17, 63]), StepEntry("b", b_ids[30 + k:31 + k], [0])])
            got[use_graphs, k] = logits.float().cpu()
        if use_graphs:
            assert any(not isinstance(key[0], int) for key in eng.graphs), "the recurring shape was not captured"
    for k in range(6):
        at = 3000 + 64 * k
        for use_graphs in (True, False):
            close(got[use_graphs, k][:3], want_a[[at, at + 17, at + 63]], "bfloat16")
            close(got[use_graphs, k][3:], want_b[[30 + k]], "bfloat16")
    assert torch.equal(got[True, 0], got[False, 0])          # both eager


def test_recorded_steps_with_the_shared_block_prompt_attention(tmp_path):
    """Five prompts of the same length, one after the other, at the 7B model's head shape: the step's shape recurs,
    so the later ones replay a captured graph, in which the prompt attention is the kernel whose waves share their
    blocks of keys (it asks the runtime for more LDS than the default at every launch, recorded or not).  Every
    prompt's logits against the plain implementation and against an engine that records nothing."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import StepEntry
    from tokenizer_amd.kernels import get_ops
    assert get_ops().lib.ta_prefill_attention_shared_plan(69, 28, 4, 128, 1536) == 11
    raw = dict(TINY["A"][0], num_hidden_layers=2, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
               intermediate_size=256, vocab_size=300, max_position_embeddings=2048, rope_theta=1000000.0)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 19, str(tmp_path / "recorded"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    prompts = [random_ids(300, 1100, 60 + i) for i in range(5)]
    rows = [0, 500, 1099]
    got = {}
    for use_graphs in (True, False):
        eng = engine_for(folder, "bfloat16", max_tokens=1152, max_requests=1, use_graphs=use_graphs)
        eng.pools.poison()
        for i, ids in enumerate(prompts):
            eng.add_request(i)
            got[use_graphs, i] = eng.step([StepEntry(i, ids, rows)]).float().cpu()
            eng.end_request(i)
        if use_graphs:
            assert any(not isinstance(key[0], int) for key in eng.graphs), "the recurring shape was not captured"
    for i, ids in enumerate(prompts):
        close(got[True, i], plain.all_logits(cfg, tensors, ids)[rows], "bfloat16")
    # The first step ran eagerly in both engines; the last one replays a graph in the first (whose big library
    # products were timed again before the capture, so their rounding may differ from the eager engine's).
    assert torch.equal(got[True, 0], got[False, 0])
    close(got[True, 4], got[False, 4], "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_first_tokens_of_a_sequence(model_folders, oracle, name, dtype):
    # Position 0 alone, then position 1 alone, then two at once: the shortest contexts there are.
    raw = TINY[name][0]
    ids = random_ids(raw["vocab_size"], 4, 7)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": ids[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": ids[1:2], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": ids[2:4], "want": [0, 1]}], "end": ["x"]}]
    eng = engine_for(model_folders[name], dtype, max_tokens=64, max_requests=2)
    eng.pools.poison()
    got = tt.run_in_process(eng, steps)
    close(got["x"], oracle(name, ids), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, oracle, tmp_path, dtype):
    # The program itself, as a child process: mixed steps, wants on some places only, a step without wants.
    name = "B"
    reqs = requests_for(name)
    steps = tt.mixed(reqs, 6)
    for step in steps[::3]:
        for entry in step["entries"]:
            entry["want"] = entry["want"][-1:]
    steps[1]["entries"][0]["want"] = []
    vocab = TINY[name][0]["vocab_size"]
    got = tt.run_program(model_folders[name], dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps), vocab)
    # Rebuild which positions were asked for.
    at = {rid: 0 for rid in reqs}
    asked = {rid: [] for rid in reqs}
    for step in steps:
        for entry in step["entries"]:
            asked[entry["id"]] += [at[entry["id"]] + w for w in entry["want"]]
            at[entry["id"]] += len(entry["tokens"])
    for rid, ids in reqs.items():
        want = oracle(name, ids)[asked[rid]]
        close(got[rid], want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [16, 48])
def test_captured_decode_steps_equal_eager_ones(model_folders, dtype, page_size):
    # The same trace with and without graph replay: decode steps of changing batch size, with a mixed step
    # (captured from its third appearance) between them, each replay checked against the eager engine.  Pages of
    # 48 tokens: a graph's context range is no whole number of pages, and still it plans its launches for the
    # range an eager step plans for.
    from tokenizer_amd.engine import StepEntry
    name = "B"
    vocab = TINY[name][0]["vocab_size"]
    engines = [engine_for(model_folders[name], dtype, max_tokens=1024, max_requests=4, use_graphs=flag,
                          page_size=page_size) for flag in (True, False)]
    assert engines[0].use_graphs and not engines[1].use_graphs
    prompts = {rid: random_ids(vocab, n, 50 + rid) for rid, n in enumerate([37, 5, 64])}
    for eng in engines:
        for rid, ids in prompts.items():
            eng.add_request(rid)
    rng_tokens = random_ids(vocab, 400, 77)
    plan = [[0], [0, 1], [0, 1, 2], "prefill", [0, 2], [1], [0, 1, 2], [0, 1, 2], "prefill", [2], [0, 1, 2]] * 3
    at = 0
    for action in plan:
        if action == "prefill":
            entries = [StepEntry(1, rng_tokens[at:at + 3], [2]), StepEntry(0, rng_tokens[at + 3:at + 4], [0])]
            at += 4
        else:
            entries = [StepEntry(rid, [rng_tokens[at + i]], [0]) for i, rid in enumerate(action)]
            at += len(action)
        got = []
        for eng in engines:
            if not all(eng.cache.seq_len(e.rid) for e in entries):          # first use: run the prompt
                eng.step([StepEntry(e.rid, prompts[e.rid], []) for e in entries if not eng.cache.seq_len(e.rid)])
            logits = eng.step(entries)
            got.append((logits.float().cpu().clone(), eng.argmax(logits)))
        torch.testing.assert_close(got[0][0], got[1][0], rtol=0, atol=0)
        assert got[0][1] == got[1][1]
    assert len(engines[0].graphs) >= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurring_step_shapes_replay_graphs_and_equal_eager_steps(model_folders, dtype, monkeypatch):
    """A step whose shape has come up before (a prompt cut into equal portions, the same mix of portions and
    decoded tokens) replays a captured graph.  Every replay is checked against an engine without graphs, with
    eager steps of other shapes and synchronisations between the replays; portions of 96 tokens take the
    vendor library's products into the graph.  When as many graphs are kept as may be, one that has not been
    replayed for a while makes room; if none is that old, the new shape runs eagerly."""
    from tokenizer_amd.engine import Engine, StepEntry
    name = "C"
    vocab = TINY[name][0]["vocab_size"]
    monkeypatch.setattr(Engine, "STEP_GRAPHS", 3)
    monkeypatch.setattr(Engine, "GRAPH_IDLE_STEPS", 6)
    from tokenizer_amd.kernels import get_ops
    monkeypatch.setattr(get_ops(), "EAGER_LIBRARY_WORK", 0)     # eager steps choose their kernels as captured ones do
    engines = [engine_for(model_folders[name], dtype, max_tokens=4096, max_requests=4, use_graphs=flag)
               for flag in (True, False)]
    ids = random_ids(vocab, 3000, 123)
    at = [0]

    def take(n):
        at[0] += n
        return ids[at[0] - n:at[0]]

    def both(make_entries):
        entries = make_entries()
        got = [eng.step(entries).float().cpu().clone() for eng in engines]
        torch.testing.assert_close(got[0], got[1], rtol=0, atol=0)
        return got[0]

    for eng in engines:
        for rid in range(4):
            eng.add_request(rid)
    for _ in range(5):                                    # equal portions of one prompt: captured at the third
        both(lambda: [StepEntry(0, take(96), [95])])
    assert any(not isinstance(key[0], int) for key in engines[0].graphs)
    both(lambda: [StepEntry(1, take(33), [32])])          # another shape, eager
    for k in range(4):                                    # a portion beside decoded tokens
        both(lambda: [StepEntry(0, take(1), [0]), StepEntry(2, take(80), [0, 79]), StepEntry(1, take(1), [0])])
        both(lambda: [StepEntry(1, take(7 + k), [])])     # shapes that never recur stay eager
    for _ in range(2):
        both(lambda: [StepEntry(3, take(96), [95])])      # the first shape again, for another request
    # Portions of 13 to 16 tokens are filled up to the same counts: one shape, one graph, whatever the length.
    before = len(engines[0].graphs)
    for n in (13, 14, 15, 16, 16, 13):
        both(lambda: [StepEntry(1, take(n), [n - 1])])
    assert len(engines[0].graphs) == before + 1
    shape_of = lambda n: Engine._shape_of([StepEntry(3, [0] * n, [n - 1])])
    assert shape_of(13) == shape_of(16) != shape_of(17)
    for n in (20, 28, 36):                                # more shapes than graphs are kept
        for _ in range(3):
            both(lambda: [StepEntry(3, take(n), [n - 1])])
    kept = [key[0] for key in engines[0].graphs if not isinstance(key[0], int)]
    assert sorted(kept) == sorted(shape_of(n) for n in (20, 28, 36))          # the idle ones made room
    for n in (19, 27, 35):
        both(lambda: [StepEntry(1, take(n), [n - 1])])    # all three in use again (by portions a little shorter) ...
    for _ in range(3):
        both(lambda: [StepEntry(1, take(44), [43])])      # ... so a further shape finds no room and runs eagerly
    kept = [key[0] for key in engines[0].graphs if not isinstance(key[0], int)]
    assert sorted(kept) == sorted(shape_of(n) for n in (20, 28, 36))
    for eng in engines:
        eng.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_decode_steps_back_to_back_equal_steps_one_by_one(model_folders, dtype, name, monkeypatch):
    """`decode_greedy` feeds each step's ids to the next on the device and reads them a step late; it must pick
    what stepping one by one picks, also across a change of graph (the context bucket is made small), and an
    early end returns exactly one step more than was asked for.  Between its steps the device itself turns a
    step's description into the next one's, and the host uploads one only where that is not what it would upload
    (a request has entered a new page or, in C's layers with a window, given one back; another graph): far fewer
    uploads than steps, and the same ids."""
    from tokenizer_amd.engine import Engine, StepEntry
    vocab = TINY[name][0]["vocab_size"]
    monkeypatch.setattr(Engine, "GRAPH_BUCKET", 48)
    monkeypatch.setattr(Engine, "NEXT_STEP_ON_DEVICE", True)
    prompts = {rid: random_ids(vocab, n, 90 + rid) for rid, n in enumerate([40, 3, 21])}
    runs = []
    for pipelined in (True, False):
        eng = engine_for(model_folders[name], dtype, max_tokens=512, max_requests=4)
        first = []
        for rid, ids in prompts.items():
            eng.add_request(rid)
            first.append(eng.argmax(eng.step([StepEntry(rid, ids, [len(ids) - 1])]))[0])
        if pipelined:
            picked = eng.decode_greedy(list(prompts), first, 30)
            assert len(eng.graphs) >= 2                      # the contexts crossed a bucket's end
            uploads = sum(graph.uploads for graph in eng.graphs.values())
            assert all(graph.advances for graph in eng.graphs.values()) and 2 <= uploads <= 20
        else:
            picked, current = [], first
            for _ in range(30):
                current = eng.argmax(eng.step([StepEntry(rid, [t], [0]) for rid, t in zip(prompts, current)]))
                picked.append(current)
        runs.append(picked)
        assert [eng.cache.seq_len(rid) for rid in prompts] == [len(ids) + 30 for ids in prompts.values()]
        # An early end: the step already launched when the answer came still counts.
        seen = []
        more = eng.decode_greedy(list(prompts), picked[-1], 10, on_step=lambda k, ids: seen.append(k) or k < 3)
        assert len(more) == 5 and seen == [0, 1, 2, 3]
        runs.append(more[:4])
        eng.cache.check_invariants()
    assert runs[0] == runs[2] and runs[1] == runs[3]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_drawn_decode_steps_back_to_back_equal_steps_one_by_one(model_folders, dtype, monkeypatch):
    """`decode_sampled` draws every step's ids on the device, feeds them to the next step there and reads them a
    step late: with the same uniform numbers it gives what stepping and drawing one by one gives, across a change
    of graph, with and without a nucleus cut; `draw` is asked once for every step that is launched, also when the
    run is ended early."""
    import random
    from tokenizer_amd.engine import Engine, StepEntry
    name = "B"
    vocab = TINY[name][0]["vocab_size"]
    monkeypatch.setattr(Engine, "GRAPH_BUCKET", 48)
    prompts = {rid: random_ids(vocab, n, 70 + rid) for rid, n in enumerate([38, 5, 20])}
    # (In the last round of cases the second request is greedy: it keeps the greedy pick among the others' draws.)
    for temperature, top_p in (([0.8, 1.3, 1.0], [1.0, 1.0, 1.0]), ([0.8, 1.3, 1.0], [0.9, 1.0, 0.5]),
                               ([0.8, 0.0, 1.0], [0.9, 1.0, 1.0])):
        warm = [row for row, t in enumerate(temperature) if t != 0]
        rng = random.Random(11)
        uniforms = [[rng.random() for _ in prompts] for _ in range(40)]
        runs = []
        for pipelined in (True, False):
            eng = engine_for(model_folders[name], dtype, max_tokens=512, max_requests=4)
            first = []
            for rid, ids in prompts.items():
                eng.add_request(rid)
                first.append(eng.argmax(eng.step([StepEntry(rid, ids, [len(ids) - 1])]))[0])
            asked = []
            draw = lambda k: (asked.append(k), (temperature, top_p, uniforms[len(asked) - 1]))[1]
            if pipelined:
                picked = eng.decode_sampled(list(prompts), first, 30, draw)
                assert len(eng.graphs) >= 2 and asked == list(range(30))
                more = eng.decode_sampled(list(prompts), picked[-1], 10, draw, on_step=lambda k, ids: k < 3)
                assert len(more) == 5 and asked[30:] == [0, 1, 2, 3, 4]
            else:
                picked, current = [], first
                for k in range(35):
                    logits = eng.step([StepEntry(rid, [t], [0]) for rid, t in zip(prompts, current)])
                    current = eng.argmax(logits)
                    drawn = eng.sample(logits, warm, [temperature[r] for r in warm], [top_p[r] for r in warm],
                                       [uniforms[k][r] for r in warm])
                    for row, token in zip(warm, drawn):
                        current[row] = token
                    picked.append(current)
                picked, more = picked[:30], picked[30:]
            runs.append(picked + more)
            assert all(0 <= t < vocab for ids in picked + more for t in ids)
            eng.cache.check_invariants()
        assert runs[0] == runs[1]
        assert len({tuple(ids) for ids in runs[0]}) > 20          # draws, not one id again and again


def sharpened(folder, out_folder, factor):
    """A copy of a model folder whose query and key projections are scaled up: attention becomes nearly
    one-hot, so a wrong key, page or window edge changes the logits by far more than any rounding."""
    import shutil
    from safetensors.torch import load_file
    from tokenizer_amd.weights import save_safetensors
    shutil.copytree(folder, out_folder)
    tensors = {k: v.clone() for k, v in load_file(folder + "/model.safetensors").items()}   # not views of a mapped file
    for name in tensors:
        if "q_proj" in name or "k_proj" in name:
            tensors[name] = (tensors[name].float() * factor).to(torch.bfloat16)
    save_safetensors(out_folder + "/model.safetensors", tensors)
    return out_folder


@pytest.mark.parametrize("name", ["B", "C"])
def test_peaked_attention_over_hundreds_of_keys(model_folders, tmp_path, name):
    # float32 only: with weights like these bfloat16 rounding alone moves the nearly one-hot choices.
    folder = sharpened(model_folders[name], str(tmp_path / "sharp"), 24.0)
    cfg, tensors = plain.load_folder(folder)
    _, tensors64 = plain.load_folder(folder, torch.float64)
    vocab, limit = cfg["vocab_size"], cfg["max_position_embeddings"]
    reqs = {f"r{i}": random_ids(vocab, min(n, limit), 90 + i) for i, n in enumerate([250, 97, 33, 180])}
    exact = {rid: plain.all_logits(cfg, tensors64, ids).float() for rid, ids in reqs.items()}
    want = {rid: plain.all_logits(cfg, tensors, ids) for rid, ids in reqs.items()}
    # Scores are 24^2 times larger here and carry that much more float32 rounding into the softmax, in any
    # implementation.  So the yardstick is the plain float32 implementation's own distance from a float64
    # run: the engine may be a few times that, no more.  A wrong key moves these logits by more than 0.05.
    plain_error = max(float((want[r] - exact[r]).abs().max()) for r in reqs)
    for steps in (tt.mixed(reqs, 8), tt.decode_tail(reqs, 32)):
        eng = engine_for(folder, "float32", max_tokens=tt.peak_tokens(steps), max_requests=4)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        for rid in reqs:
            err = float((got[rid] - exact[rid]).abs().max())
            assert err <= 4 * plain_error + 2e-5, f"engine off by {err}, plain float32 by {plain_error}"
    # The sharpening matters: the same engine run on the original weights is far from these logits.
    eng = engine_for(model_folders[name], "float32", max_tokens=1024, max_requests=4)
    other = tt.run_in_process(eng, tt.whole(reqs))
    assert max(float((other[r] - want[r]).abs().max()) for r in reqs) > 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_far_token_moves_the_last_logits_as_the_plain_model_says(model_folders, tmp_path, dtype):
    """In both dtypes, through the whole engine: with attention sharpened (not to one-hot: bfloat16 rounding must
    not decide), one token changed some two hundred positions back moves the last logits by several times the
    bfloat16 bound.  The engine has to show the same move, decoding token by token and in mixed batches with
    reused pages: a key read from a wrong page, a split of the key range left out or a block table row mixed up
    would lose it, where the nearly uniform attention of the other tests' weights would hide that."""
    name = "B"
    folder = sharpened(model_folders[name], str(tmp_path / "sharp"), 8.0)
    cfg, tensors64 = plain.load_folder(folder, torch.float64)
    vocab = cfg["vocab_size"]
    ids = random_ids(vocab, 250, 91)
    base = plain.all_logits(cfg, tensors64, ids).float()
    moves = []
    for at in (2, 5, 9, 14, 20, 33, 47):
        other = list(ids)
        other[at] = (other[at] + 101) % vocab
        moved = plain.all_logits(cfg, tensors64, other).float()
        moves.append((float((moved[-16:] - base[-16:]).abs().max()), at, other, moved))
    effect, at, other, moved = max(moves, key=lambda item: item[0])
    bound = TOL[dtype] * max(1.0, float(base.abs().max()))
    assert effect > 5 * TOL["bfloat16"], "the weights and inputs should make one far token matter"
    reqs = {"base": ids, "moved": other, "beside": random_ids(vocab, 120, 92)}
    for steps in (tt.decode_tail(reqs, 32), tt.mixed(reqs, 12, max_live=3)):
        eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=3)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        close(got["base"], base, dtype)
        close(got["moved"], moved, dtype)
        shown = got["moved"][-16:] - got["base"][-16:]
        assert float((shown - (moved[-16:] - base[-16:])).abs().max()) <= 2 * bound
        assert float(shown.abs().max()) >= effect - 2 * bound
        eng.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_points(model_folders, tmp_path, dtype):
    import subprocess
    import sys
    from tokenizer_amd.engine import GenerateParams, generate, greedy_tokens
    name = "B"
    cfg, tensors = plain.load_folder(model_folders[name])
    prompt = random_ids(cfg["vocab_size"], 11, 5)
    want = plain.greedy_generate(cfg, tensors, prompt, 8)
    eng = engine_for(model_folders[name], dtype, num_pages=8, max_requests=2)
    out = generate(eng, prompt, GenerateParams.greedy(8))
    if dtype == "float32":
        assert out.tokens == want and greedy_tokens(eng, prompt, 8) == want
    assert out.completion_tokens == 8 and out.reason.value == "MaxTokens" and out.prefill > 0 and out.decode > 0
    # The command line: ids in, ids out (the folder has no tokenizer.json), the reference's lines on stderr.
    root = tt.ROOT
    run = subprocess.run([sys.executable, f"{root}/bin/qwen-infer", "--model", model_folders[name], "--dtype", dtype,
                          "--max-tokens", "8", "--token-ids", " ".join(map(str, prompt))],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert f"prompt ids ({len(prompt)}): {prompt}" in run.stderr
    assert "max_tokens 8 temperature 0 top_p 1 seed 0 eos []" in run.stderr
    assert f"generated ids: {out.tokens}" in run.stderr and "stop: MaxTokens" in run.stderr
    assert "tok/s (8 tokens, KV cache, total" in run.stderr
    assert run.stdout.split() == [str(t) for t in out.tokens]
    # A warm request: the command line queues it through the scheduler, `generate` drives the step function itself;
    # both draw the same ids from the request's own seed.
    warm = GenerateParams(max_tokens=7, temperature=0.9, top_p=0.8, seed=11)
    alone = generate(eng, prompt, warm)
    run = subprocess.run([sys.executable, f"{root}/bin/qwen-infer", "--model", model_folders[name], "--dtype", dtype,
                          "--max-tokens", "7", "--temperature", "0.9", "--top-p", "0.8", "--seed", "11",
                          "--num-blocks", "8", "--token-ids", " ".join(map(str, prompt))],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert "max_tokens 7 temperature 0.9 top_p 0.8 seed 11 eos []" in run.stderr
    assert f"generated ids: {alone.tokens}" in run.stderr
    # A prompt the pool cannot hold is answered with the scheduler's message, not a traceback.
    run = subprocess.run([sys.executable, f"{root}/bin/qwen-infer", "--model", model_folders[name], "--dtype", dtype,
                          "--num-blocks", "2", "--token-ids", " ".join(map(str, random_ids(cfg["vocab_size"], 60, 6)))],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 1 and "error: kv pool has 2 blocks of 16; this sequence needs" in run.stderr


def test_warm_requests_draw_on_the_device_as_they_would_alone(model_folders):
    # Temperature and nucleus draws in a batch of the scheduler equal the same requests run one by one:
    # the uniform numbers are the request's own, and the sampling kernel sees only that request's row.
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig, generate
    name = "A"
    vocab = TINY[name][0]["vocab_size"]
    prompts = [random_ids(vocab, n, 70 + n) for n in (4, 9, 2, 17)]
    params = [GenerateParams(max_tokens=10, temperature=t, top_p=p, seed=s)
              for t, p, s in ((1.3, 0.95, 5), (0.7, 1.0, 6), (1.3, 0.5, 5), (0.0, 1.0, 1))]
    eng = engine_for(model_folders[name], "float32", num_pages=32, max_requests=4)
    sched = Scheduler(eng, SchedulerConfig(num_blocks=32, max_batch_size=4))
    rids = [sched.add_request(p, q) for p, q in zip(prompts, params)]
    results = sched.run()
    solo = engine_for(model_folders[name], "float32", num_pages=32, max_requests=1)
    for rid, prompt, q in zip(rids, prompts, params):
        assert results[rid].tokens == generate(solo, prompt, q).tokens
    assert len({tuple(results[r].tokens) for r in rids}) == 4
    again = generate(solo, prompts[0], params[0]).tokens
    other = generate(solo, prompts[0], GenerateParams(max_tokens=10, temperature=1.3, top_p=0.95, seed=6)).tokens
    assert again == results[rids[0]].tokens and other != again
    sched.assert_idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_draws_of_a_replayed_step_equal_eager_draws(model_folders, dtype):
    # A batch in which every request draws with a temperature: its decode steps replay a captured graph, and the
    # sampler's launches over that graph's logits replay one as well (with and without the nucleus rounds).  The
    # tokens equal those of an engine that captures nothing, step after step.
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig
    name = "B"
    vocab = TINY[name][0]["vocab_size"]
    prompts = [random_ids(vocab, n, 90 + n) for n in (6, 6, 6)]
    for cuts in ((0.9, 0.5, 0.97), (1.0, 1.0, 1.0)):
        params = [GenerateParams(max_tokens=14, temperature=t, top_p=p, seed=s)
                  for t, p, s in zip((1.2, 0.8, 2.0), cuts, (3, 4, 5))]
        tokens = {}
        for use_graphs in (True, False):
            eng = engine_for(model_folders[name], dtype, num_pages=32, max_requests=4, use_graphs=use_graphs)
            sched = Scheduler(eng, SchedulerConfig(num_blocks=32, max_batch_size=4))
            rids = [sched.add_request(p, q) for p, q in zip(prompts, params)]
            results = sched.run()
            tokens[use_graphs] = [results[rid].tokens for rid in rids]
            if use_graphs:
                assert any(graph.draws for graph in eng.graphs.values())
        assert tokens[True] == tokens[False]
        assert all(len(t) == 14 for t in tokens[True])


REAL_SIZES = {
    # Layer sizes of the three model sizes the benchmarks name, cut to two layers and a small vocabulary.
    "0.5b": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864),
    "1.5b": dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960),
    "7b": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944),
}


@pytest.mark.parametrize("size", list(REAL_SIZES))
def test_layers_of_real_sizes(tmp_path, size, monkeypatch):
    # The kernels at the widths, head sizes and group sizes of the real models: prompts in portions, decode
    # steps alone and in a batch (fused and unfused kernels, captured graphs), against the plain implementation.
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    raw = dict(TINY["A"][0], num_hidden_layers=2, vocab_size=1000, max_position_embeddings=512,
               tie_word_embeddings=(size != "7b"), **REAL_SIZES[size])
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 11, str(tmp_path / size), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    reqs = {f"r{i}": random_ids(1000, n, 20 + i) for i, n in enumerate([150, 47, 80])}
    want = {rid: plain.all_logits(cfg, tensors, ids) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for steps in (tt.mixed(reqs, 2), tt.decode_tail(reqs, 24)):
            eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4)
            eng.pools.poison()
            got = tt.run_in_process(eng, steps)
            for rid in reqs:
                close(got[rid], want[rid], dtype)
    if raw["hidden_size"] // raw["num_attention_heads"] == 128:
        # Heads of 128: with hundreds of tiles in a step the prompt kernel whose waves share each block of keys
        # takes over; these prompts are far too short for that, so it is asked for.
        from tokenizer_amd.kernels import get_ops
        monkeypatch.setattr(get_ops(), "prefill_shared", 1)
        steps = tt.mixed(reqs, 2)
        eng = engine_for(folder, "bfloat16", max_tokens=tt.peak_tokens(steps), max_requests=4)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        for rid in reqs:
            close(got[rid], want[rid], "bfloat16")
        monkeypatch.setattr(get_ops(), "prefill_shared", 0)
    # A decode batch of 20 requests takes the kernels for more than 16 rows.
    from tokenizer_amd.engine import StepEntry
    eng = engine_for(folder, "bfloat16", max_tokens=64 * 20, max_requests=20)
    prompts = [random_ids(1000, 30 + i, 40 + i) for i in range(20)]
    for rid, ids in enumerate(prompts):
        eng.add_request(rid)
        eng.step([StepEntry(rid, ids[:-1], [])])
    logits = eng.step([StepEntry(rid, ids[-1:], [0]) for rid, ids in enumerate(prompts)]).float().cpu()
    for rid, ids in enumerate(prompts):
        close(logits[rid:rid + 1], plain.all_logits(cfg, tensors, ids)[-1:], "bfloat16")


ODD_SIZES = {
    # Sizes away from every tile: an inner width that is no multiple of eight, odd vocabularies, head sizes from
    # 16 to 256, one to eighteen query heads per kv head, a model wider than the norm-folding kernels take.
    "inner100": dict(num_hidden_layers=1, hidden_size=112, num_attention_heads=7, num_key_value_heads=7,
                     intermediate_size=100, vocab_size=1001),
    "inner300_mqa": dict(num_hidden_layers=2, hidden_size=144, num_attention_heads=3, num_key_value_heads=1,
                         intermediate_size=300, vocab_size=517, tie_word_embeddings=False, rms_norm_eps=1e-5),
    "group18": dict(num_hidden_layers=1, hidden_size=288, num_attention_heads=18, num_key_value_heads=1,
                    intermediate_size=204, vocab_size=777),
    "head256": dict(num_hidden_layers=1, hidden_size=256, num_attention_heads=1, num_key_value_heads=1,
                    intermediate_size=36, vocab_size=99),
    "wide": dict(num_hidden_layers=1, hidden_size=2304, num_attention_heads=18, num_key_value_heads=6,
                 intermediate_size=1004, vocab_size=500),
    "window_inner44": dict(num_hidden_layers=3, hidden_size=320, num_attention_heads=2, num_key_value_heads=2,
                           intermediate_size=44, vocab_size=129, use_sliding_window=True, sliding_window=33,
                           max_window_layers=1),
}


@pytest.mark.parametrize("size", list(ODD_SIZES))
def test_sizes_away_from_every_tile(tmp_path, size):
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    raw = dict(TINY["A"][0], max_position_embeddings=512, **ODD_SIZES[size])
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 13, str(tmp_path / size), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    reqs = {f"r{i}": random_ids(raw["vocab_size"], n, 30 + i) for i, n in enumerate([70, 33, 100, 9])}
    want = {rid: plain.all_logits(cfg, tensors, ids) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for steps in (tt.mixed(reqs, 6), tt.decode_tail(reqs, 32)):
            eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4)
            eng.pools.poison()
            got = tt.run_in_process(eng, steps)
            for rid in reqs:
                close(got[rid], want[rid], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_like_layers_make_the_recorded_calls_of_the_first_again(model_folders, name, dtype):
    """Eager steps record the library calls of one layer and make them again for the like layers after it, with
    their weights' and pages' addresses put in place.  The logits equal, bit for bit, those of an engine whose
    layers all run their own Python: mixed batches with reused pages, and decode steps (whose fused layers hand
    nothing on, so the first layer already serves the rest).  Configuration C has a full layer and three with a
    window: the second layer is the one that is recorded for the two after it."""
    reqs = requests_for(name)
    n_layers = TINY[name][0]["num_hidden_layers"]
    for steps in (tt.mixed(reqs, 9), tt.decode_tail(reqs, 12)):
        logits, repeated = [], []
        for repeat in (True, False):
            eng = engine_for(model_folders[name], dtype, max_tokens=tt.peak_tokens(steps), max_requests=4,
                             use_graphs=False)
            eng.model.decoder.repeat_layers = repeat
            eng.pools.poison()
            logits.append(tt.run_in_process(eng, steps))
            repeated.append(eng.model.decoder.layers_repeated)
        for rid in reqs:
            assert torch.equal(logits[0][rid], logits[1][rid]), rid
        assert repeated[1] == 0
        # Every step repeats the layers behind the recorded one of each make: all but two (the first hands on what
        # it was not handed), or all but one where a layer hands nothing on.
        assert repeated[0] >= len(steps) * (n_layers - 2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_model_under_one_engine_after_another(model_folders, oracle, dtype):
    """A model outlives its engines (a benchmark makes one engine per batch size over one model): the second and
    third engines have pools of other sizes at other addresses, and the first is gone (collected) when they run.
    Their eager mixed steps repeat recorded layers and still equal, bit for bit, an engine whose layers all run
    their own Python, and the plain model."""
    import gc
    from tokenizer_amd.engine import Engine, load_model
    name = "C"
    reqs = requests_for(name)
    steps = tt.mixed(reqs, 21)
    model = load_model(model_folders[name], dtype)
    plain_engine = engine_for(model_folders[name], dtype, max_tokens=tt.peak_tokens(steps), max_requests=4, use_graphs=False)
    plain_engine.model.decoder.repeat_layers = False
    want = tt.run_in_process(plain_engine, steps)
    for extra_pages in (0, 7, 3, 11, 0, 5):
        eng = Engine(model, num_pages=-(-tt.peak_tokens(steps) // 16) + extra_pages, max_requests=4, use_graphs=False)
        eng.pools.poison()
        before = model.decoder.layers_repeated
        got = tt.run_in_process(eng, steps)
        assert model.decoder.layers_repeated > before
        for rid, ids in reqs.items():
            assert torch.equal(got[rid], want[rid]), (rid, extra_pages)
            close(got[rid], oracle(name, ids), dtype)
        del eng
        gc.collect()
        torch.cuda.empty_cache()


def test_a_layer_named_twice_and_a_layer_on_anothers_pages_are_repeated_rightly(tmp_path):
    """The order of layers is data: a schedule that runs a layer twice and lets a layer read another layer's pages
    (without writing) gives the same logits whether the like layers repeat recorded calls or run on their own."""
    import dataclasses
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config, register_architecture, registered_architectures
    from tokenizer_amd.models.qwen2 import qwen2_spec
    from tokenizer_amd.parts.spec import ScheduleEntry

    class TwiceConfig(Qwen2Config):
        pass

    def twice_spec(cfg):
        spec = qwen2_spec(cfg)
        order = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(1), ScheduleEntry(3),
                 ScheduleEntry(2, cache_of=3), ScheduleEntry(3, cache_of=3), ScheduleEntry(1))
        return dataclasses.replace(spec, architecture="TwiceQwen2ForCausalLM", schedule=order)

    if "TwiceQwen2ForCausalLM" not in registered_architectures():
        register_architecture("TwiceQwen2ForCausalLM", TwiceConfig, twice_spec)
    raw = dict(TINY["B"][0], architectures=["TwiceQwen2ForCausalLM"], num_hidden_layers=4, max_window_layers=4)
    folder = ta.write_random_model(TwiceConfig.from_dict(raw), 3, str(tmp_path / "twice"), norm_spread=0.3)
    reqs = {f"r{i}": random_ids(raw["vocab_size"], n, 70 + i) for i, n in enumerate([40, 7, 90, 33])}
    for dtype in ("float32", "bfloat16"):
        steps = tt.mixed(reqs, 2)
        got = []
        for repeat in (True, False):
            eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4, use_graphs=False)
            eng.model.decoder.repeat_layers = repeat
            eng.pools.poison()
            got.append(tt.run_in_process(eng, steps))
            assert (eng.model.decoder.layers_repeated > 0) == repeat
        for rid in reqs:
            assert torch.equal(got[0][rid], got[1][rid]), rid
            assert torch.isfinite(got[0][rid]).all()


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations_pages_and_traces(tmp_path, seed):
    """Configurations drawn at random (head sizes in steps of 16, any number of heads and groups, inner widths and
    vocabularies that are no power of two, windows on some layers, one to three layers), pages of 16, 32 or 48
    tokens, one of the ways to cut requests into steps, 32-bit or bfloat16: every logit against the plain model,
    nothing left over.  With every step recorded and replayed at its first sight (odd seeds), the replays also equal
    an engine that records nothing, bit for bit."""
    import random
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import Engine
    from tokenizer_amd.kernels import get_ops
    rng = random.Random(5000 + seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    n_kv = rng.choice([1, 2, 3, 5])
    n_q = n_kv * rng.choice([1, 2, 3, 4, 7, 8] if d <= 64 else [1, 2, 4])
    layers = rng.choice([1, 2, 3])
    window = rng.random() < 0.4
    max_pos = rng.choice([160, 300, 520])
    raw = dict(TINY["A"][0], num_hidden_layers=layers, hidden_size=n_q * d, num_attention_heads=n_q,
               num_key_value_heads=n_kv, intermediate_size=rng.choice([40, 100, 136, 272, 500]),
               vocab_size=rng.choice([97, 256, 333, 1000]), rope_theta=rng.choice([10000.0, 1e6]),
               rms_norm_eps=rng.choice([1e-6, 1e-5]), tie_word_embeddings=rng.random() < 0.5,
               max_position_embeddings=max_pos, use_sliding_window=window,
               sliding_window=rng.choice([5, 21, 64, 100]) if window else max_pos,
               max_window_layers=rng.randrange(0, layers + 1) if window else layers)
    page_size = rng.choice([16, 16, 32, 48])
    dtype = rng.choice(["float32", "bfloat16"])
    kind = rng.choice(["mixed", "portions", "tail"])
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), seed, str(tmp_path / "drawn"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    lens = [min(n, max_pos) for n in rng.sample([1, 2, 9, 17, 40, 64, 65, 100, 130, 150, 257, 400], 5)]
    reqs = {f"r{i}": random_ids(raw["vocab_size"], n, 10 * seed + i) for i, n in enumerate(lens)}
    steps = {"mixed": lambda: tt.mixed(reqs, seed), "portions": lambda: tt.portions(reqs, seed),
             "tail": lambda: tt.decode_tail(reqs)}[kind]()
    recorded = seed % 2 == 1
    before = (Engine.GRAPH_AFTER, Engine.STEP_GRAPHS, get_ops().EAGER_LIBRARY_WORK)
    try:
        if recorded:
            Engine.GRAPH_AFTER, Engine.STEP_GRAPHS = 1, 10 ** 6
            get_ops().EAGER_LIBRARY_WORK = 0          # eager steps choose their products as recorded ones do
        eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4, page_size=page_size)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        for rid, ids in reqs.items():
            close(got[rid], plain.all_logits(cfg, tensors, ids), dtype)
        eng.cache.check_invariants()
        assert not eng.cache.requests
        if recorded:
            assert eng.graphs
            eager = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4, page_size=page_size,
                               use_graphs=False)
            eager.pools.poison()
            again = tt.run_in_process(eager, steps)
            for rid in reqs:
                assert torch.equal(got[rid], again[rid]), rid
    finally:
        Engine.GRAPH_AFTER, Engine.STEP_GRAPHS, get_ops().EAGER_LIBRARY_WORK = before


def test_the_whole_model_at_half_a_billion_parameters(tmp_path):
    # All 24 layers and the vocabulary of 151,936 at Qwen2.5-0.5B sizes, random weights: prompts in portions beside
    # decoded tokens and with their last tokens one by one, in 32-bit and in bfloat16, against the plain implementation.
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    raw = dict(TINY["A"][0], num_hidden_layers=24, vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=True, max_position_embeddings=32768, sliding_window=32768, max_window_layers=24,
               **REAL_SIZES["0.5b"])
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 0, str(tmp_path / "half_b"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    reqs = {f"r{i}": random_ids(raw["vocab_size"], n, 50 + i) for i, n in enumerate([150, 70, 33])}
    want = {rid: plain.all_logits(cfg, tensors, ids) for rid, ids in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for steps in (tt.mixed(reqs, 3), tt.decode_tail(reqs, 8)):
            eng = engine_for(folder, dtype, max_tokens=tt.peak_tokens(steps), max_requests=4)
            eng.pools.poison()
            got = tt.run_in_process(eng, steps)
            for rid in reqs:
                close(got[rid], want[rid], dtype)
            del eng


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [8, 32, 48])
def test_other_page_sizes(model_folders, oracle, dtype, page_size):
    # Pages of 32 and 48 tokens take the matrix-core attention kernels as pages of 16 do; pages of 8 (no multiple
    # of a key tile) go to the generic kernel.  Mixed batches with reused pages, configuration C with its window.
    for name in ("B", "C"):
        reqs = requests_for(name)
        steps = tt.mixed(reqs, 7)
        live = tt.peak_tokens(steps)
        eng = engine_for(model_folders[name], dtype, max_tokens=live, page_size=page_size, max_requests=4)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        for rid, ids in reqs.items():
            close(got[rid], oracle(name, ids), dtype)
        eng.cache.check_invariants()
        assert not eng.cache.requests


@pytest.mark.parametrize("size", ["inner100", "group18", "wide", "window_inner44"])
def test_decode_batches_of_dozens_at_sizes_away_from_every_tile(tmp_path, size):
    # Decode batches of 20 and 64 requests (the kernels for 17 to 64 rows: K cut over workgroups with the parts
    # left to the norm, two column blocks, the rotation epilogue with the rows in shares) at odd sizes, two steps
    # each, in bfloat16 and in 32-bit, against the plain implementation.
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import StepEntry
    raw = dict(TINY["A"][0], max_position_embeddings=512, **ODD_SIZES[size])
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 17, str(tmp_path / size), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    for dtype in ("bfloat16", "float32"):
        for batch in (20, 64):
            eng = engine_for(folder, dtype, max_tokens=64 * batch, max_requests=batch)
            prompts = [random_ids(raw["vocab_size"], 3 + (7 * i) % 40, 200 + i) for i in range(batch)]
            for rid, ids in enumerate(prompts):
                eng.add_request(rid)
                eng.step([StepEntry(rid, ids[:-1], [])])
            for _ in range(2):
                logits = eng.step([StepEntry(rid, ids[-1:], [0]) for rid, ids in enumerate(prompts)]).float().cpu()
                for rid, ids in enumerate(prompts):
                    close(logits[rid:rid + 1], plain.all_logits(cfg, tensors, ids)[-1:], dtype)
                prompts = [ids + [int(logits[rid].argmax())] for rid, ids in enumerate(prompts)]
